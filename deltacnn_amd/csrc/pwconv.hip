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
//                     Used while the filter fragments of a wavefront fit in registers (up to
//                     8 channel tiles x 5 reduction steps); larger layers keep the two-launch
//                     form, whose channel split over many workgroups streams big filters fast
#include "epilogue.hpp"

namespace dc {
namespace {

__device__ __forceinline__ half8_t zero8() { return half8_t{0, 0, 0, 0, 0, 0, 0, 0}; }

struct PwP {
    int P, Ci, Co, ci_p, co_tiles;
};

// S = reduction steps per memory round trip (chunk): all fragment loads of S steps are in
// flight together; the host picks the smallest S in {1, 2, 4, 8} that covers a wavefront's
// share of the reduction, so most layers finish in a single chunk.
//
// ADD fuses the residual sum of a DCAdd layer behind the convolution: with a = residual delta
// (mask Ma) and b = convolution output rounded to fp16 (mask Mb = input mask),
// out = fma(b, wb, a * wa) on pixels of Ma | Mb, each term present only where its mask is set --
// the same operations, in the same order and precision, as the stand-alone add kernel.
struct ResP {
    const half_t *res;
    const int32_t *mask;
    float wa, wb;
};

template <bool KSPLIT, int S, bool ADD>
__global__ void __launch_bounds__(256)
pw_mfma_kernel(PwP p, const half_t *__restrict__ in, const half_t *__restrict__ wp,
               const half_t *__restrict__ bias, half_t *__restrict__ out,
               const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, ResP rp) {
    constexpr int NT = 4;
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
    bool on[NT], on_r[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        px[nt] = blockIdx.x * 64 + nt * 16 + l16;
        const int m = mask[min(px[nt], p.P - 1)];
        on[nt] = px[nt] < p.P && m != 0;
        on_r[nt] = false;
        if (ADD) on_r[nt] = px[nt] < p.P && rp.mask[min(px[nt], p.P - 1)] != 0;
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
        any |= ballot(on[nt] || on_r[nt]) != 0;
    }
    if (cb == 0 && wave == 0 && kq == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            if (px[nt] < p.P) out_mask[px[nt]] = (on[nt] || on_r[nt]) ? 1 : 0;
    }
    if (!any) return;
    const int co = ct * 16 + kq * 4;  // Cout % 4 == 0: a lane's 4 channels are all in or all out
    half4_t res[NT];
    if (ADD) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            res[nt] = *reinterpret_cast<const half4_t *>(
                rp.res + (size_t)(on_r[nt] ? px[nt] : 0) * p.Co + min(co, p.Co - 4));
    }

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
        // No zero-fill is needed: columns of inactive pixels are never stored, and where a step
        // reaches past Cin the packed filter holds zeros while the clamped address re-reads
        // finite values of the same pixel.
#pragma unroll
        for (int i = 0; i < S; ++i) {
            if (s0 + i * stride < ksteps) {  // wave-uniform
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    if (nt_on[nt])  // wave-uniform
                        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], x[i][nt], acc[nt], 0, 0, 0);
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
    if (co >= p.Co) return;
    float4_t bv = {0.f, 0.f, 0.f, 0.f};
    if (bias != nullptr) {
        const half4_t b = *reinterpret_cast<const half4_t *>(bias + co);
        bv = float4_t{float(b[0]), float(b[1]), float(b[2]), float(b[3])};
    }
    const half_t wa = half_t(rp.wa), wb = half_t(rp.wb);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (!(on[nt] || on_r[nt]) || (KSPLIT && nt != wave)) continue;
        const float4_t r = acc[nt] + bv;
        half4_t o = half4_t{half_t(r[0]), half_t(r[1]), half_t(r[2]), half_t(r[3])};
        if (ADD) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                half_t sum = on_r[nt] ? half_t(res[nt][i] * wa) : half_t(0);
                if (on[nt]) sum = fma_t(o[i], wb, sum);
                o[i] = sum;
            }
        }
        *reinterpret_cast<half4_t *>(out + (size_t)px[nt] * p.Co + co) = o;
    }
}

// --------------------------------------------------------------- fused conv + act/trunc
// Workgroup = NW wavefronts x 16 pixels x all output channels; wavefront w owns channel tiles
// w, w + NW, ... (at most CTW of them).  KS bounds the reduction steps: the input fragments of
// the 16 pixels stay in registers for the whole kernel and every loop is fully unrolled without
// branches (surplus steps multiply zero fragments, surplus tiles are computed and dropped), so
// the filter stream of a wavefront is one uninterrupted run of loads.  Requires Cout % 4 == 0.
// Pass 1 of the epilogue: conv output v (rounded to fp16), T = trunc + v, S = T + prev,
// D = act(S) - act(prev), one rounding each; collects the keep statistics of this lane.
template <int CTW, int ACT>
__device__ __forceinline__ void pw_epilogue_stats(const float4_t (&acc)[CTW], const half4_t (&q)[CTW],
                                                  const half4_t (&tr)[CTW], half4_t (&v)[CTW],
                                                  const half_t *__restrict__ bias, bool on, int wave,
                                                  int NW, int kq, const PwP &p, half_t thr, bool &hit,
                                                  float &sq) {
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        if (ct >= p.co_tiles) break;  // wave-uniform: surplus tiles of the last wavefronts
        const int co = ct * 16 + kq * 4;
        const bool live = co < p.Co;
        float4_t r = acc[j];
        if (bias != nullptr && live) {
            const half4_t b = *reinterpret_cast<const half4_t *>(bias + co);
            r += float4_t{float(b[0]), float(b[1]), float(b[2]), float(b[3])};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[j][i] = half_t(r[i]);
            const half_t t = tr[j][i] + v[j][i];
            const half_t s = t + q[j][i];
            const half_t d = act_apply<half_t>(s, ACT) - act_apply<half_t>(q[j][i], ACT);
            if (live && on) {
                hit |= tabs(d) > thr;
                sq += float(d) * float(d);
            }
        }
    }
}

// Pass 2: recompute T, S, D (a handful of ALU operations, cheaper than keeping them in
// registers across the workgroup barrier) and write the kept / dropped state.
template <int CTW, int ACT>
__device__ __forceinline__ void pw_epilogue_store(const half4_t (&q)[CTW], const half4_t (&tr)[CTW],
                                                  const half4_t (&v)[CTW], bool keep, int wave, int NW,
                                                  int kq, int px, const PwP &p,
                                                  half_t *__restrict__ out, half_t *__restrict__ prev,
                                                  half_t *__restrict__ trunc) {
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        if (ct >= p.co_tiles) break;  // wave-uniform
        const int co = ct * 16 + kq * 4;
        if (co >= p.Co) continue;
        const size_t off = (size_t)px * p.Co + co;
        half4_t t, s, d;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            t[i] = tr[j][i] + v[j][i];
            s[i] = t[i] + q[j][i];
            d[i] = act_apply<half_t>(s[i], ACT) - act_apply<half_t>(q[j][i], ACT);
        }
        if (keep) {
            *reinterpret_cast<half4_t *>(prev + off) = s;
            *reinterpret_cast<half4_t *>(out + off) = d;
            *reinterpret_cast<half4_t *>(trunc + off) = half4_t{0, 0, 0, 0};
        } else {
            *reinterpret_cast<half4_t *>(trunc + off) = t;
        }
    }
}

#define DC_ACT_SWITCH(act, CALL)                                                \
    switch (act) {                                                              \
        case DC_ACT_RELU: { constexpr int A = DC_ACT_RELU; CALL; } break;       \
        case DC_ACT_RELU6: { constexpr int A = DC_ACT_RELU6; CALL; } break;     \
        case DC_ACT_LEAKY: { constexpr int A = DC_ACT_LEAKY; CALL; } break;     \
        case DC_ACT_SIGMOID: { constexpr int A = DC_ACT_SIGMOID; CALL; } break; \
        case DC_ACT_SWISH: { constexpr int A = DC_ACT_SWISH; CALL; } break;     \
        default: { constexpr int A = DC_ACT_LINEAR; CALL; } break;              \
    }

// Workgroup = NW wavefronts x 16 pixels x all output channels; wavefront w owns channel tiles
// w, w + NW, ... (at most CTW of them).  KS bounds the reduction steps.  Every loop is fully
// unrolled without branches (surplus steps multiply zero fragments, surplus tiles are computed
// and dropped).  The filter fragments of a wavefront are requested in AB batches: the first
// together with the mask words, the second together with the input fragments and the cached
// state, so the kernel is two memory round trips, the MFMAs, one barrier and the stores.
// Requires Cout % 4 == 0.
template <int NW, int CTW, int KS, int AB>
__global__ void __launch_bounds__(NW * WAVE)
pw_act_mfma_kernel(PwP p, const half_t *__restrict__ in, const half_t *__restrict__ wp,
                   const half_t *__restrict__ bias, half_t *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                   half_t *__restrict__ prev, half_t *__restrict__ trunc, float thr_f, int act,
                   int mode) {
    static_assert(CTW % AB == 0, "filter batches must divide the tiles of a wavefront");
    constexpr int JB = CTW / AB;
    __shared__ float s_stat[NW][16];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int kvalid = kq * 8;
    const int ksteps = p.ci_p >> 5;
    const int px = blockIdx.x * 16 + l16;
    const int m = mask[min(px, p.P - 1)];
    half8_t a[CTW][KS];
    // round trip 1: mask word + first batch of filter fragments (they do not depend on the
    // mask; a workgroup without active pixels wastes a few cached KB)
#pragma unroll
    for (int j = 0; j < JB; ++j) {
        const int ct = min(wave + j * NW, p.co_tiles - 1);
        const half_t *wrow = wp + (size_t)(ct * 16 + l16) * p.ci_p + kvalid;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            a[j][s] = *reinterpret_cast<const half8_t *>(wrow + (min(s, ksteps - 1) << 5));
    }
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
        for (int s = 0; s < KS; ++s) DC_PIN(a[j][s]);
    const bool on = px < p.P && m != 0;
    if (ballot(on) == 0) {  // same 16 pixels in every wavefront: the whole workgroup leaves
        if (wave == 0 && kq == 0 && px < p.P) out_mask[px] = 0;
        return;
    }
    // round trip 2: remaining filter fragments, input fragments and cached state of this
    // lane's (pixel, 4 channel) cells; inactive pixels all point at pixel 0, their loads share
    // one cache line and are dropped
#pragma unroll
    for (int j = JB; j < CTW; ++j) {
        const int ct = min(wave + j * NW, p.co_tiles - 1);
        const half_t *wrow = wp + (size_t)(ct * 16 + l16) * p.ci_p + kvalid;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            a[j][s] = *reinterpret_cast<const half8_t *>(wrow + (min(s, ksteps - 1) << 5));
    }
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
    for (int j = JB; j < CTW; ++j)
#pragma unroll
        for (int s = 0; s < KS; ++s) DC_PIN(a[j][s]);
#pragma unroll
    for (int s = 0; s < KS; ++s) DC_PIN(x[s]);
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        DC_PIN(q[j]);
        DC_PIN(tr[j]);
    }
    // no zero-fill: see pw_mfma_kernel (inactive columns are dropped, padded filter is zero)
    float4_t acc[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s)
            if (s < ksteps)  // uniform
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j][s], x[s], acc[j], 0, 0, 0);
    }
    const half_t thr = half_t(thr_f);
    half4_t v[CTW];
    bool hit = false;
    float sq = 0.f;
    DC_ACT_SWITCH(act, (pw_epilogue_stats<CTW, A>(acc, q, tr, v, bias, on, wave, NW, kq, p, thr, hit, sq)));
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
    DC_ACT_SWITCH(act, (pw_epilogue_store<CTW, A>(q, tr, v, keep, wave, NW, kq, px, p, out, prev, trunc)));
}

}  // namespace

bool pointwise_eligible(const dc_geometry &g, int dtype) {
    return dtype == DC_F16 && g.groups == 1 && g.in_c % 8 == 0 && g.in_c >= 8 && g.out_c % 4 == 0 &&
           g.kernel_h == 1 &&
           g.kernel_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
           g.pad_left == 0 && g.pad_bottom == 0 && g.pad_right == 0;
}

// Reduction steps above which the convolution-only kernel splits the reduction over the
// wavefronts of a workgroup.  The fused kernel only takes much shorter reductions, so a layer
// gets the same summation order with and without the fused epilogue.
constexpr int PW_KSPLIT_STEPS = 10;

hipError_t launch_pointwise(const dc_geometry &g, const void *in, const void *packed,
                            const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                            const ActEpilogue *epi, bool *epilogue_done, const Residual *res,
                            hipStream_t s) {
    PwP p;
    p.P = g.batch * g.in_h * g.in_w;
    p.Ci = g.in_c;
    p.Co = g.out_c;
    p.ci_p = (g.in_c + 31) / 32 * 32;
    p.co_tiles = ceil_div(g.out_c, 16);
    const int ksteps = p.ci_p / 32;
    *epilogue_done = false;
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    // Fused epilogue where a workgroup can own all output channels of 16 pixels cheaply: few
    // channel tiles per wavefront and a short reduction, so that all filter fragments of a
    // wavefront live in registers.
    const bool fusable = res == nullptr && epi != nullptr && epi->mode >= 0 && g.out_c % 4 == 0 && al8(epi->prev) &&
                         al8(epi->trunc) && al8(out);
    if (fusable) {
        dim3 grid(ceil_div(p.P, 16));
        const int act = epi->act < 0 ? 0 : epi->act;
#define DC_GO(NW, CTW, KS, AB)                                                                       \
    do {                                                                                             \
        pw_act_mfma_kernel<NW, CTW, KS, AB><<<grid, NW * WAVE, 0, s>>>(                              \
            p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, \
            out_mask, (half_t *)epi->prev, (half_t *)epi->trunc, epi->thr, act, epi->mode);          \
        *epilogue_done = true;                                                                       \
        return hipGetLastError();                                                                    \
    } while (0)
        // Only maps with enough pixels to occupy the GPU with 16-pixel workgroups: a wavefront
        // issues one instruction per 4 cycles, so a small map handled by a few fat workgroups is
        // slower than the two-launch form whose channel split spreads over many wavefronts.
        if (p.P > 1024) {
            const int ctw = ceil_div(p.co_tiles, 4);
            if (ctw <= 2 && ksteps <= 1) DC_GO(4, 2, 1, 1);
            if (ctw <= 3 && ksteps <= 1) DC_GO(4, 3, 1, 1);
            if (ctw <= 4 && ksteps <= 1) DC_GO(4, 4, 1, 1);
            if (ctw <= 2 && ksteps <= 3) DC_GO(4, 2, 3, 1);
            if (ctw <= 4 && ksteps <= 3) DC_GO(4, 4, 3, 1);
            if (ctw <= 8 && ksteps <= 1) DC_GO(4, 8, 1, 1);
            if (ctw <= 8 && ksteps <= 2) DC_GO(4, 8, 2, 1);
        }
#undef DC_GO
    }
    const bool ksplit = ksteps > PW_KSPLIT_STEPS;
    dim3 grid(ceil_div(p.P, 64), ksplit ? p.co_tiles : ceil_div(p.co_tiles, 4));
    const int per_wave = ksplit ? ceil_div(ksteps, 4) : ksteps;
    ResP rp{nullptr, nullptr, 1.f, 1.f};
    if (res != nullptr) rp = ResP{(const half_t *)res->values, res->mask, res->wa, res->wb};
#define DC_PW(KS, SS)                                                                                \
    do {                                                                                             \
        if (res != nullptr)                                                                          \
            pw_mfma_kernel<KS, SS, true><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask, rp); \
        else                                                                                         \
            pw_mfma_kernel<KS, SS, false><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask, rp); \
    } while (0)
    if (ksplit) {
        if (per_wave <= 4) DC_PW(true, 4); else DC_PW(true, 8);
    } else {
        if (per_wave <= 1) DC_PW(false, 1);
        else if (per_wave <= 2) DC_PW(false, 2);
        else if (per_wave <= 4) DC_PW(false, 4);
        else DC_PW(false, 8);
    }
#undef DC_PW
    return hipGetLastError();
}

}  // namespace dc
