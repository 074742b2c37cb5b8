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

}  // namespace dc
