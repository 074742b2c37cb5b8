// Output-tile machinery shared by the convolution and pooling kernels: window geometry, the
// tap -> input coordinate map, and the mask phase that dilates the input mask over the window
// and compacts the active output pixels of an 8x8 tile.
#pragma once

#include "common.hpp"

namespace dc {

constexpr int TILE = 8;           // output tile edge
constexpr int TILE_PX = TILE * TILE;

struct ConvP {
    int B, Hi, Wi, Ci, Ho, Wo, Co;
    int Kh, Kw, sh, sw, dh, dw, pt, pl;
    int ci_g, co_g;   // channels per group
    int w_co;         // filter row length (Cout, padded to even for swizzled fp16)
    int swz;          // fp16 channel-pair swizzle present
};

// Input coordinate feeding output coordinate `o` through tap `k`; false if there is none.
template <bool TR>
__device__ __forceinline__ bool tap_src(int o, int k, int stride, int dil, int pad, int limit,
                                        int &i) {
    if (TR) {
        int t = o + pad - k * dil;
        if (t < 0) return false;
        i = t / stride;
        return (t - i * stride) == 0 && i < limit;
    }
    i = o * stride - pad + k * dil;
    return i >= 0 && i < limit;
}

// Phase 1 shared by all conv kernels.  Returns the number of active output pixels of the tile;
// s_list[0..n) holds their (oy << 16 | ox).  Must be called by the whole workgroup.
template <bool TR>
__device__ __forceinline__ int tile_mask_phase(const ConvP &p, const int32_t *__restrict__ mask,
                                               int32_t *__restrict__ out_mask, int b, int ty0,
                                               int tx0, bool write_mask, int *s_list, int *s_n) {
    if (threadIdx.x < WAVE) {
        int oy = ty0 + (threadIdx.x >> 3), ox = tx0 + (threadIdx.x & 7);
        bool inb = oy < p.Ho && ox < p.Wo;
        bool upd = false;
        if (inb) {
            const int32_t *m = mask + (size_t)b * p.Hi * p.Wi;
            for (int ky = 0; ky < p.Kh; ++ky) {
                int iy;
                if (!tap_src<TR>(oy, ky, p.sh, p.dh, p.pt, p.Hi, iy)) continue;
                for (int kx = 0; kx < p.Kw; ++kx) {
                    int ix;
                    if (!tap_src<TR>(ox, kx, p.sw, p.dw, p.pl, p.Wi, ix)) continue;
                    upd |= m[iy * p.Wi + ix] != 0;
                }
            }
            if (write_mask) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = upd ? 1 : 0;
        }
        int n;
        int rank = wave_rank(upd, n);
        if (upd) s_list[rank] = (oy << 16) | ox;
        if (threadIdx.x == 0) *s_n = n;
    }
    __syncthreads();
    return *s_n;
}

// Phase 1 of the MFMA convolution: the mask phase and the source table in one pass.  Lane i of
// the first wavefront owns output pixel i of the 8x8 tile; it requests the mask words of all its
// taps at once (nine at a time, clamped addresses), so the whole phase is one memory round trip.
// Results in LDS: s_list[0..n) = active output pixels (oy << 16 | ox); s_src[tap * 64 + slot] =
// input pixel index read by compacted pixel `slot` through `tap`, or -1 (out of bounds, inactive,
// or slot >= n); s_taplist[0..*s_ntaps) = the taps used by at least one pixel, ascending.
// The tile's pixels are (ty0 + i * ystep, tx0 + j * xstep), i, j = 0..7: a transposed
// convolution takes the stride as step, so that all pixels of a tile share one stride phase
// and hence one set of (K / stride)^2 taps.  Returns n.  Must be called by the whole workgroup
// (K2 <= 64).
template <bool TR>
__device__ __forceinline__ int tile_front(const ConvP &p, const int32_t *__restrict__ mask,
                                          int32_t *__restrict__ out_mask, int b, int ty0, int tx0,
                                          int ystep, int xstep, bool write_mask, int *s_list,
                                          int *s_src, int *s_taplist, int *s_ntaps, int *s_n) {
    if (threadIdx.x < WAVE) {
        const int K2 = p.Kh * p.Kw;
        const int oy = ty0 + (threadIdx.x >> 3) * ystep, ox = tx0 + (threadIdx.x & 7) * xstep;
        const bool inb = oy < p.Ho && ox < p.Wo;
        const int32_t *m = mask + (size_t)b * p.Hi * p.Wi;
        unsigned long long bits = 0;
        for (int t0 = 0; t0 < K2; t0 += 9) {
            int word[9];
            bool ok[9];
#pragma unroll
            for (int j = 0; j < 9; ++j) {
                const int tap = min(t0 + j, K2 - 1);
                const int ky = tap / p.Kw, kx = tap - ky * p.Kw;
                int iy = 0, ix = 0;
                ok[j] = inb && t0 + j < K2 && tap_src<TR>(oy, ky, p.sh, p.dh, p.pt, p.Hi, iy) &&
                        tap_src<TR>(ox, kx, p.sw, p.dw, p.pl, p.Wi, ix);
                word[j] = m[ok[j] ? iy * p.Wi + ix : 0];
            }
#pragma unroll
            for (int j = 0; j < 9; ++j)
                if (ok[j] && word[j] != 0) bits |= 1ull << (t0 + j);
        }
        const bool upd = bits != 0;
        if (inb && write_mask) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = upd ? 1 : 0;
        int n;
        const int rank = wave_rank(upd, n);
        // active pixels take slots 0..n-1 in lane order, the others fill n..63 with -1 rows
        const int slot = upd ? rank : n + (int)threadIdx.x - rank;
        if (upd) s_list[rank] = (oy << 16) | ox;
        for (int tap = 0; tap < K2; ++tap) {
            int src = -1;
            if ((bits >> tap) & 1ull) {
                const int ky = tap / p.Kw, kx = tap - ky * p.Kw;
                int iy, ix;
                tap_src<TR>(oy, ky, p.sh, p.dh, p.pt, p.Hi, iy);
                tap_src<TR>(ox, kx, p.sw, p.dw, p.pl, p.Wi, ix);
                src = iy * p.Wi + ix;
            }
            s_src[tap * TILE_PX + slot] = src;
        }
        unsigned long long used = bits;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) used |= __shfl_xor(used, o, WAVE);
        if ((int)threadIdx.x < K2 && ((used >> threadIdx.x) & 1ull))
            s_taplist[__popcll(used & ((1ull << threadIdx.x) - 1ull))] = threadIdx.x;
        if (threadIdx.x == 0) {
            *s_n = n;
            *s_ntaps = __popcll(used);
        }
    }
    __syncthreads();
    return *s_n;
}

// The resident-filter form of the LDS-halo kernel (convres.hip): thin layers on large maps.  The
// arguments after the geometry are the launch plan of conv_lds_mfma_kernel for the layer.
bool resident_conv_eligible(const dc_geometry &g, int hal_h, int hal_w, int ltx, int lty, int kcc, int rl,
                            int ksl, int ncw);
hipError_t launch_resident_conv(const dc_geometry &g, const ConvP &p, int hal_h, int hal_w, int ltx, int lty, int kcc,
                                int rl, int ksl, int ncw, const void *in, const void *packed, const void *bias,
                                void *out, const int32_t *mask, int32_t *out_mask, int dtype, hipStream_t s);

}  // namespace dc
