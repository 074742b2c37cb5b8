// Delta convolution and delta transposed convolution.
//
// Every kernel works on an 8x8 tile of output pixels per workgroup:
//   1. one lane per output pixel ORs the input mask over the filter window (the dilated
//      output mask), writes it, and the active output pixels of the tile are compacted with
//      ballot + popcount rank; a tile without active pixels ends here;
//   2. only the compacted pixels are computed.  Inactive or out-of-bounds inputs contribute
//      zero by selection (their memory is never read).
//
// conv_direct_kernel  any dtype / kernel / stride / dilation / groups, VALU, fp32 accumulate
// conv_mfma_kernel    fp16, groups == 1, Cin % 8 == 0: implicit GEMM on
//                     v_mfma_f32_16x16x32_f16 with rows = output channels (packed filter
//                     [Cout][tap][Cin]) and columns = compacted pixels (NHWC rows), so both
//                     operands are 16-byte row loads and the accumulator tile stores 4
//                     consecutive channels per lane
#include "tile.hpp"

namespace dc {
namespace {

// ---------------------------------------------------------------------------------- direct
// Threads run along output channels (coalesced filter reads and output writes); 256/COT
// pixel groups each take PB compacted pixels at a time, so one filter value is reused PB
// times from a register while the input values are wave-uniform broadcast loads.
template <typename T, bool TR>
__global__ void __launch_bounds__(256)
conv_direct_kernel(ConvP p, const T *__restrict__ in, const T *__restrict__ filter,
                   const T *__restrict__ bias, T *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, int COT) {
    constexpr int PB = 4;
    __shared__ int s_list[TILE_PX];
    __shared__ int s_n;
    const int b = blockIdx.z;
    const int n = tile_mask_phase<TR>(p, mask, out_mask, b, blockIdx.y * TILE, blockIdx.x * TILE,
                                      true, s_list, &s_n);
    if (n == 0) return;

    const int pg = threadIdx.x / COT, cl = threadIdx.x % COT, PG = 256 / COT;
    const int K2 = p.Kh * p.Kw;
    const T *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    for (int co = cl; co < p.Co; co += COT) {
        const int cin0 = (co / p.co_g) * p.ci_g;
        const int wsw = p.swz ? (co & 1) : 0;
        for (int base = pg * PB; base < n; base += PG * PB) {
            float acc[PB];
            int oy[PB], ox[PB];
#pragma unroll
            for (int j = 0; j < PB; ++j) {
                acc[j] = 0.f;
                int code = base + j < n ? s_list[base + j] : -1;
                oy[j] = code >> 16;
                ox[j] = code & 0xffff;
                if (code < 0) oy[j] = -1;
            }
            for (int ky = 0; ky < p.Kh; ++ky) {
                for (int kx = 0; kx < p.Kw; ++kx) {
                    int ip[PB];
                    bool any = false;
#pragma unroll
                    for (int j = 0; j < PB; ++j) {
                        ip[j] = -1;
                        int iy, ix;
                        if (oy[j] >= 0 && tap_src<TR>(oy[j], ky, p.sh, p.dh, p.pt, p.Hi, iy) &&
                            tap_src<TR>(ox[j], kx, p.sw, p.dw, p.pl, p.Wi, ix) &&
                            mb[iy * p.Wi + ix] != 0) {
                            ip[j] = iy * p.Wi + ix;
                            any = true;
                        }
                    }
                    if (!any) continue;
                    const int tap = ky * p.Kw + kx;
                    for (int cg = 0; cg < p.ci_g; ++cg) {
                        float w = float(filter[((size_t)(cg ^ wsw) * K2 + tap) * p.w_co + co]);
#pragma unroll
                        for (int j = 0; j < PB; ++j)
                            if (ip[j] >= 0) acc[j] += float(inb[(size_t)ip[j] * p.Ci + cin0 + cg]) * w;
                    }
                }
            }
            float bv = bias != nullptr ? float(bias[co]) : 0.f;
#pragma unroll
            for (int j = 0; j < PB; ++j)
                if (oy[j] >= 0)
                    out[(((size_t)b * p.Ho + oy[j]) * p.Wo + ox[j]) * p.Co + co] = T(acc[j] + bv);
        }
    }
}

// ------------------------------------------------------------------------------------ MFMA
// One work item = one 16(channels) x 16(pixels) accumulator tile with the full reduction over
// taps and input channels; the items of a workgroup (channel tiles of its channel block x
// pixel sub-tiles of its compacted list) are dealt round-robin to its four wavefronts.
template <bool TR>
__global__ void __launch_bounds__(256)
conv_mfma_kernel(ConvP p, const half_t *__restrict__ in, const half_t *__restrict__ wp,
                 const half_t *__restrict__ bias, half_t *__restrict__ out,
                 const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, int co_blocks,
                 int co_tiles_per_block, int ci_p) {
    __shared__ int s_list[TILE_PX];
    __shared__ int s_n;
    const int b = blockIdx.z / co_blocks;
    const int cb = blockIdx.z % co_blocks;
    const int n = tile_mask_phase<TR>(p, mask, out_mask, b, blockIdx.y * TILE, blockIdx.x * TILE,
                                      cb == 0, s_list, &s_n);
    if (n == 0) return;

    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;  // row/column inside the tile, k-quarter
    const int K2 = p.Kh * p.Kw;
    const int n_tiles = (n + 15) >> 4;
    const int co_tiles = (p.Co + 15) >> 4;
    const int ct0 = cb * co_tiles_per_block;
    const int ct_end = min(ct0 + co_tiles_per_block, co_tiles);
    const int items = (ct_end - ct0) * n_tiles;
    const half_t *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const bool pointwise = !TR && K2 == 1 && p.sh == 1 && p.sw == 1 && p.pt == 0 && p.pl == 0;

    for (int item = wave; item < items; item += 4) {
        const int ct = ct0 + item / n_tiles, nt = item % n_tiles;
        const int pix = nt * 16 + l16;
        const int code = pix < n ? s_list[pix] : -1;
        const int oy = code >> 16, ox = code & 0xffff;
        const half_t *wrow = wp + (size_t)(ct * 16 + l16) * K2 * ci_p + kq * 8;
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
        for (int ky = 0; ky < p.Kh; ++ky) {
            for (int kx = 0; kx < p.Kw; ++kx) {
                int ipix = -1;
                if (code >= 0) {
                    if (pointwise) {
                        ipix = oy * p.Wi + ox;
                    } else {
                        int iy, ix;
                        if (tap_src<TR>(oy, ky, p.sh, p.dh, p.pt, p.Hi, iy) &&
                            tap_src<TR>(ox, kx, p.sw, p.dw, p.pl, p.Wi, ix) &&
                            mb[iy * p.Wi + ix] != 0)
                            ipix = iy * p.Wi + ix;
                    }
                }
                if (ballot(ipix >= 0) == 0) continue;  // no pixel of this sub-tile uses the tap
                const half_t *xrow = inb + (size_t)(ipix < 0 ? 0 : ipix) * p.Ci + kq * 8;
                const half_t *wt = wrow + (size_t)(ky * p.Kw + kx) * ci_p;
                for (int k0 = 0; k0 < ci_p; k0 += 32) {
                    half8_t a = *reinterpret_cast<const half8_t *>(wt + k0);
                    half8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
                    if (ipix >= 0 && k0 + kq * 8 < p.Ci) x = *reinterpret_cast<const half8_t *>(xrow + k0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, x, acc, 0, 0, 0);
                }
            }
        }
        // lane holds channels ct*16 + kq*4 + {0..3} of pixel `pix`
        if (code >= 0) {
            const int co = ct * 16 + kq * 4;
            half_t *o = out + (((size_t)b * p.Ho + oy) * p.Wo + ox) * p.Co + co;
            if (co + 3 < p.Co && (p.Co & 3) == 0) {
                half4_t r;
#pragma unroll
                for (int i = 0; i < 4; ++i) r[i] = half_t(acc[i] + (bias ? float(bias[co + i]) : 0.f));
                *reinterpret_cast<half4_t *>(o) = r;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (co + i < p.Co) o[i] = half_t(acc[i] + (bias ? float(bias[co + i]) : 0.f));
            }
        }
    }
}

// One-time relayout of a reference-layout fp16 filter [Cin pad 2][K][K][Cout pad 2] (channel
// pairs swizzled: W[ci][co] is stored at row ci ^ (co & 1)) into [Cout pad 16][K][K][Cin pad 32].
__global__ void pack_filter_kernel(const half_t *__restrict__ f, half_t *__restrict__ wp, int Ci,
                                   int Co, int K2, int w_co, int ci_p, int co_p) {
    const size_t total = (size_t)co_p * K2 * ci_p;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        int ci = int(i % ci_p);
        int tap = int((i / ci_p) % K2);
        int co = int(i / ((size_t)ci_p * K2));
        half_t v = half_t(0);
        if (ci < Ci && co < Co) v = f[((size_t)(ci ^ (co & 1)) * K2 + tap) * w_co + co];
        wp[i] = v;
    }
}

inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

inline bool mfma_eligible(const dc_geometry &g, int dtype) {
    return dtype == DC_F16 && g.groups == 1 && g.in_c % 8 == 0 && g.in_c >= 8;
}

ConvP make_params(const dc_geometry &g, int dtype) {
    ConvP p;
    p.B = g.batch; p.Hi = g.in_h; p.Wi = g.in_w; p.Ci = g.in_c;
    p.Ho = g.out_h; p.Wo = g.out_w; p.Co = g.out_c;
    p.Kh = g.kernel_h; p.Kw = g.kernel_w; p.sh = g.stride_h; p.sw = g.stride_w;
    p.dh = g.dilation_h; p.dw = g.dilation_w; p.pt = g.pad_top; p.pl = g.pad_left;
    p.ci_g = g.in_c / g.groups;
    p.co_g = g.out_c / g.groups;
    const bool depthwise = g.groups > 1;
    p.swz = (dtype == DC_F16 && !depthwise) ? 1 : 0;
    p.w_co = p.swz ? g.out_c + (g.out_c & 1) : g.out_c;
    return p;
}

}  // namespace

int64_t packed_filter_bytes(const dc_geometry &g, int dtype, bool transposed) {
    (void)transposed;
    if (!mfma_eligible(g, dtype)) return 0;
    return (int64_t)round_up(g.out_c, 16) * g.kernel_h * g.kernel_w * round_up(g.in_c, 32) * 2;
}

hipError_t launch_pack_filter(const dc_geometry &g, const void *filter, void *packed, int dtype,
                              bool transposed, hipStream_t s) {
    (void)transposed;
    if (!mfma_eligible(g, dtype)) return hipSuccess;
    const int K2 = g.kernel_h * g.kernel_w;
    const int ci_p = round_up(g.in_c, 32), co_p = round_up(g.out_c, 16);
    const size_t total = (size_t)co_p * K2 * ci_p;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    pack_filter_kernel<<<blocks, 256, 0, s>>>((const half_t *)filter, (half_t *)packed, g.in_c,
                                              g.out_c, K2, g.out_c + (g.out_c & 1), ci_p, co_p);
    return hipGetLastError();
}

hipError_t launch_conv(const dc_geometry &g, const void *in, const void *filter,
                       const void *packed, const void *bias, void *out, const int32_t *mask,
                       int32_t *out_mask, int dtype, bool transposed, const ActEpilogue *epi,
                       hipStream_t s) {
    ConvP p = make_params(g, dtype);
    const int tx = ceil_div(g.out_w, TILE), ty = ceil_div(g.out_h, TILE);
    if (packed != nullptr && mfma_eligible(g, dtype)) {
        const int co_tiles = ceil_div(g.out_c, 16);
        const int tiles_per_block = 4;  // one channel tile per wavefront and pixel sub-tile
        const int co_blocks = ceil_div(co_tiles, tiles_per_block);
        dim3 grid(tx, ty, g.batch * co_blocks);
        const int ci_p = round_up(g.in_c, 32);
        if (transposed)
            conv_mfma_kernel<true><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask, co_blocks, tiles_per_block, ci_p);
        else
            conv_mfma_kernel<false><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)packed, (const half_t *)bias, (half_t *)out, mask, out_mask, co_blocks, tiles_per_block, ci_p);
    } else {
        dim3 grid(tx, ty, g.batch);
        int COT = pow2_ceil(g.out_c);
        if (COT > 256) COT = 256;
        if (dtype == DC_F32) {
            if (transposed)
                conv_direct_kernel<float, true><<<grid, 256, 0, s>>>(p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, COT);
            else
                conv_direct_kernel<float, false><<<grid, 256, 0, s>>>(p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, COT);
        } else {
            if (transposed)
                conv_direct_kernel<half_t, true><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)filter, (const half_t *)bias, (half_t *)out, mask, out_mask, COT);
            else
                conv_direct_kernel<half_t, false><<<grid, 256, 0, s>>>(p, (const half_t *)in, (const half_t *)filter, (const half_t *)bias, (half_t *)out, mask, out_mask, COT);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || epi == nullptr) return e;
    return launch_activate_truncate(out, epi->prev, epi->trunc, out_mask, epi->thr, epi->act,
                                    epi->mode, g.batch * g.out_h * g.out_w, g.out_c, dtype, s);
}

}  // namespace dc
