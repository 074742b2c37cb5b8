// K x K delta convolution on the matrix cores for THIN layers on LARGE maps: the filter stays in
// registers and a workgroup walks over many output tiles.
//
// conv_lds_mfma_kernel (conv.hip) gives every 8x8 output tile a workgroup of its own, which
// streams its share of the filter from L2 -- for 64 -> 64 channels 73 KB per tile against 13 KB
// of input halo and 8 KB of output.  On a map of thousands of tiles that stream is most of the
// kernel's traffic and time.  Here a workgroup is launched once per compute-unit slot and loops
// over tiles (tile = blockIdx.x, blockIdx.x + gridDim.x, ...): the filter fragments of each
// wavefront's reduction steps (at most RES_MAX_STEPS steps x R channel tiles) are loaded before
// the loop and stay in registers, the step table is built once, and per tile only the mask words,
// the halo and the outputs move.  The mask words and halo rows of the NEXT tile are requested
// before the reduction of the current one (unconditionally, from clamped addresses, and selected
// by the mask afterwards), so the memory round trips of a tile hide behind the previous tile's
// matrix instructions instead of heading its dependency chain.
//
// Everything else is the algorithm of conv_lds_mfma_kernel for a plain (not transposed)
// convolution whose input channels fit one LDS chunk: halo staged in LDS with inactive and
// out-of-bounds pixels as zeros, mask dilation and compaction of the tile's updated pixels by the
// first wavefront, wavefront = (channel group cw, reduction slice kz), slice kz taking steps
// kz, kz + KS, ... in ascending order, partial sums of the slices added in ascending slice order,
// one rounding after the bias.  An output element is accumulated by the same instruction sequence
// in both kernels, so they agree bit for bit.
#include <algorithm>
#include <type_traits>

#include "epilogue.hpp"
#include "tile.hpp"

namespace dc {
namespace {

constexpr int RES_MAX_STEPS = 10;   // reduction steps per wavefront that stay in registers
constexpr int RES_MAX_HALO = 1024;  // halo pixels (table in LDS)
constexpr int RES_MAX_TABLE = 96;   // reduction steps of a tile (taps x channel steps)

struct ResP {
    int ci_p, hal_h, hal_w, kcc, lgv;
    int pitch;  // pixels per halo row in LDS (>= hal_w)
    int ltx, lty, tiles;  // tiles per row / column of a map, tiles in all (batch included)
};

template <typename E, int R, int KS, int NSW, int SU>
__global__ void __launch_bounds__(8 * WAVE)
conv_res_mfma_kernel(ConvP p, ResP q, const E *__restrict__ in, const E *__restrict__ wp,
                     const E *__restrict__ bias, E *__restrict__ out,
                     const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NT = 4;
    extern __shared__ __align__(16) unsigned char s_halo[];
    __shared__ int s_hpix[RES_MAX_HALO];
    __shared__ int2 s_step[RES_MAX_TABLE];
    __shared__ int s_list[TILE_PX];
    __shared__ int s_n;
    const int cb = blockIdx.y;
    const int tid = threadIdx.x, nthr = blockDim.x, nw = nthr / WAVE;
    const int wv = wave_id(), lane = lane_id();
    const int ncw = nw / KS, cw = wv % ncw, kz = wv / ncw;
    const int l16 = lane & 15, kq = lane >> 4;
    const int hal_h = q.hal_h, hal_w = q.hal_w, hpx = hal_h * hal_w;
    const int co_tiles = (p.Co + 15) >> 4;
    const int ksteps = q.ci_p >> 5;  // == q.kcc: all input channels in one chunk
    const int K2 = p.Kh * p.Kw;
    const int nsteps = K2 * ksteps;
    const int row = q.kcc * 64 + 16;  // bytes per staged halo pixel
    auto tap_off = [&](int a, int b2) { return a * p.dh * hal_w + b2 * p.dw; };        // in the pixel table
    auto tap_lds = [&](int a, int b2) { return a * p.dh * q.pitch + b2 * p.dw; };      // in the staged halo

    // step table: LDS byte offset of a step's input fragment relative to a pixel's halo origin
    // and its fragment offset in the packed filter; the same for every tile
    for (int j = tid; j < nsteps; j += nthr) {
        const int tap = j / ksteps, ks = j - tap * ksteps;
        const int ta = tap / p.Kw, tb = tap - ta * p.Kw;
        s_step[j] = int2{tap_lds(ta, tb) * row + ks * 64, (tap * ksteps + ks) * 512};
    }
    __syncthreads();
    // the wavefront's filter fragments, resident for the whole kernel
    E8 a[NSW][R];
    int xoff[NSW];
#pragma unroll
    for (int i = 0; i < NSW; ++i) {
        const int2 e = s_step[min(i * KS + kz, nsteps - 1)];
        xoff[i] = e.x;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const unsigned wfrag = (unsigned)min((cb * ncw + cw) * R + r, co_tiles - 1) * K2 * ksteps * 512 + lane * 8;
            a[i][r] = *reinterpret_cast<const E8 *>(wp + (wfrag + (unsigned)e.y));
        }
    }
    E bv[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int co = ((cb * ncw + cw) * R + r) * 16 + kq * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) bv[r][i] = bias != nullptr ? bias[min(co + i, p.Co - 1)] : E(0);
    }
    // Staging: 2^lgv lanes per halo pixel, SU pixels per lane (host: SU * hstep >= hpx).  A lane
    // requests the mask word and its 16 bytes of each of its pixels from clamped coordinates.
    const int sv = tid & ((1 << q.lgv) - 1), hstep = nthr >> q.lgv;
    const int tiles_per_map = q.ltx * q.lty;
    E8 val[SU];
    int word[SU], hpixel[SU];  // mask word; pixel index in the map, -1 outside of it
    int hyx[SU];               // the lane's halo pixels (row << 16 | column): the same for every tile
#pragma unroll
    for (int u = 0; u < SU; ++u) {
        const int hp = min((tid >> q.lgv) + u * hstep, hpx - 1);
        const int hy = hp / hal_w;
        hyx[u] = (hy << 16) | (hp - hy * hal_w);
    }
    const int cst = min(sv * 8, p.Ci - 8);
    auto request = [&](int tile) {
        const int b = tile / tiles_per_map, tr = tile - b * tiles_per_map;
        const int iy0 = (tr / q.ltx) * TILE * p.sh - p.pt, ix0 = (tr % q.ltx) * TILE * p.sw - p.pl;
        const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
        const E *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci + cst;
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const int iy = iy0 + (hyx[u] >> 16), ix = ix0 + (hyx[u] & 0xffff);
            const bool ok = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
            const int px = min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1);
            hpixel[u] = ok ? px : -1;
            word[u] = mb[px];
            val[u] = *reinterpret_cast<const E8 *>(inb + (unsigned)(px * p.Ci));
        }
    };
    if ((int)blockIdx.x < q.tiles) request(blockIdx.x);

    for (int tile = blockIdx.x; tile < q.tiles; tile += gridDim.x) {
        const int b = tile / tiles_per_map, tr = tile - b * tiles_per_map;
        const int ty0 = (tr / q.ltx) * TILE, tx0 = (tr % q.ltx) * TILE;
        __syncthreads();  // the previous tile's readers of the halo, the table and the list are done
        {   // what was requested for this tile: table entry (first lane of a pixel) and halo bytes
            const bool vok = sv < q.kcc * 4 && sv * 8 < p.Ci;
#pragma unroll
            for (int u = 0; u < SU; ++u) {
                const int hp = (tid >> q.lgv) + u * hstep;
                const bool on = hpixel[u] >= 0 && word[u] != 0;
                if (hp < hpx) {
                    if (sv == 0) s_hpix[hp] = on ? hpixel[u] : -1;
                    if (sv < q.kcc * 4)
                        *reinterpret_cast<E8 *>(s_halo + ((hyx[u] >> 16) * q.pitch + (hyx[u] & 0xffff)) * row + sv * 16) =
                            keep8(val[u], vok && on);
                }
            }
        }
        __syncthreads();
        if (tid < WAVE) {  // dilate the mask over the window, compact the updated pixels
            const int ly = tid >> 3, lx = tid & 7;
            const int oy = ty0 + ly, ox = tx0 + lx;
            const bool inside = oy < p.Ho && ox < p.Wo;
            bool upd = false;
            const int base = ly * p.sh * hal_w + lx * p.sw;
            for (int ta = 0; ta < p.Kh; ++ta)
                for (int tb = 0; tb < p.Kw; ++tb) upd |= s_hpix[base + tap_off(ta, tb)] >= 0;
            upd = upd && inside;
            if (inside && cb == 0) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = upd ? 1 : 0;
            int n;
            const int rank = wave_rank(upd, n);
            if (upd) s_list[rank] = tid;
            if (tid == 0) s_n = n;
        }
        __syncthreads();
        const int n = s_n;
        // the next tile's mask words and halo rows travel while this one is contracted
        if (tile + (int)gridDim.x < q.tiles) request(tile + gridDim.x);
        if (n == 0) continue;  // the same for every wavefront

        const int n_tiles = (n + 15) >> 4;
        int hbase[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int slot = nt * 16 + l16;
            const int loc = slot < n ? s_list[slot] : 0;
            hbase[nt] = ((loc >> 3) * p.sh * q.pitch + (loc & 7) * p.sw) * row + kq * 16;
        }
        float4_t acc[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[r][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
        auto reduce = [&](auto nta_tag) {
            constexpr int NTA = decltype(nta_tag)::value;
#pragma unroll
            for (int i = 0; i < NSW; ++i) {
                if (i * KS + kz >= nsteps) break;  // wave-uniform
                E8 x[NTA];
#pragma unroll
                for (int nt = 0; nt < NTA; ++nt) x[nt] = *reinterpret_cast<const E8 *>(s_halo + hbase[nt] + xoff[i]);
#pragma unroll
                for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r][nt] = Elem16<E>::mfma(a[i][r], x[nt], acc[r][nt]);
            }
        };
        switch (n_tiles) {
            case 1: reduce(std::integral_constant<int, 1>{}); break;
            case 2: reduce(std::integral_constant<int, 2>{}); break;
            case 3: reduce(std::integral_constant<int, 3>{}); break;
            default: reduce(std::integral_constant<int, 4>{}); break;
        }
        if (KS > 1) {  // partial sums of the reduction slices meet in LDS (the halo is no longer needed)
            float4_t *s_part = reinterpret_cast<float4_t *>(s_halo);
            __syncthreads();
            if (kz > 0) {
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        s_part[((((kz - 1) * ncw + cw) * R + r) * NT + nt) * WAVE + lane] = acc[r][nt];
            }
            __syncthreads();
            if (kz > 0) continue;  // these wavefronts wait at the top of the next tile
#pragma unroll
            for (int s = 1; s < KS; ++s)  // ascending slice order
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc[r][nt] += s_part[((((s - 1) * ncw + cw) * R + r) * NT + nt) * WAVE + lane];
        }
        E *otile = out + (((size_t)b * p.Ho + ty0) * p.Wo + tx0) * p.Co;  // the tile's first output pixel
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int ct = (cb * ncw + cw) * R + r;
            if (ct >= co_tiles) continue;
            const int co = ct * 16 + kq * 4;  // lane holds channels co .. co + 3 of pixel (nt, l16)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int pix = nt * 16 + l16;
                if (pix >= n) continue;
                const int loc = s_list[pix];
                E *o = otile + (unsigned)(((loc >> 3) * p.Wo + (loc & 7)) * p.Co + co);
                E4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = E(acc[r][nt][i] + float(bv[r][i]));
                if (co + 3 < p.Co && (p.Co & 3) == 0) {
                    *reinterpret_cast<E4 *>(o) = v;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (co + i < p.Co) o[i] = v[i];
                }
            }
        }
    }
}

}  // namespace

// Pixels per halo row in LDS.  A 16-pixel tile of a dense output tile is two rows of eight
// pixels; with a staged pixel of 16 bytes x an odd count, its 16 fragment reads hit distinct
// bank groups when the second row starts 8 (mod 16) pixels behind the first.
static int halo_pitch(const dc_geometry &g, int hal_w) {
    if (g.stride_w != 1) return hal_w;
    int pitch = hal_w;
    while (pitch % 16 != 8) ++pitch;
    return pitch;
}

// Layers the resident-filter kernel takes, given the arrangement conv_lds_mfma_kernel would use
// (R channel tiles per wavefront, KS reduction slices, ncw channel groups, kcc channel steps per
// LDS chunk): all input channels in one chunk of at least two steps, at most RES_MAX_STEPS
// reduction steps per wavefront, LDS within the default limit, and enough tiles that walking
// over them pays.
bool resident_conv_eligible(const dc_geometry &g, int hal_h, int hal_w, int ltx, int lty, int kcc, int rl,
                            int ksl, int ncw) {
    const int ksteps = (g.in_c + 31) / 32;
    const int nsteps = g.kernel_h * g.kernel_w * ksteps;
    const int co_tiles = ceil_div(g.out_c, 16);
    const int cbl = ceil_div(co_tiles, ncw * rl);
    // Measured on 8 x 512 x 512 maps against conv_lds_mfma_kernel: 17-20 % faster where the filter
    // takes two channel steps (64 -> 64: 399 -> 319 us, 64 -> 32: 352 -> 280 us), no gain or a loss
    // for a single channel step, whose filter of a few KB was never the cost (32 -> 64 stride 2:
    // 67 -> 70 us; 16 -> 16 on 544 x 960: 19.6 -> 22.8 us).
    if (kcc < 2) return false;
    // (four slices x two channel tiles x ten steps of fragments would not fit the register file)
    if (kcc != ksteps || nsteps > RES_MAX_TABLE || ceil_div(nsteps, ksl) > (ksl == 4 ? 5 : RES_MAX_STEPS)) return false;
    if (!((rl == 1 && ksl == 1) || (rl == 2 && (ksl == 1 || ksl == 2 || ksl == 4)))) return false;
    const int hpx = hal_h * hal_w;
    if (hpx > RES_MAX_HALO) return false;
    const size_t lds = std::max((size_t)hal_h * halo_pitch(g, hal_w) * (kcc * 64 + 16), (size_t)(ksl - 1) * ncw * rl * 4 * 1024);
    if (lds > (48u << 10)) return false;  // + 5 KB of tables: within the 64 KB a workgroup gets without asking
    const int hstep = (ncw * ksl * WAVE) >> log2i(pow2_ceil(kcc * 4));
    if (ceil_div(hpx, hstep) > 12) return false;  // halo rows a lane keeps in flight
    // (offsets within one map of the batch are computed in 32 bits)
    if ((int64_t)g.in_h * g.in_w * g.in_c >= (1ll << 31) || (int64_t)g.out_h * g.out_w * g.out_c >= (1ll << 31)) return false;
    return (int64_t)ltx * lty * g.batch * cbl >= 2048;
}

template <typename E>
static hipError_t resident_t(const dc_geometry &g, const ConvP &p, int hal_h, int hal_w, int ltx, int lty, int kcc,
                             int rl, int ksl, int ncw, const void *in, const void *packed, const void *bias,
                             void *out, const int32_t *mask, int32_t *out_mask, hipStream_t s) {
    const int co_tiles = ceil_div(g.out_c, 16);
    const int cbl = ceil_div(co_tiles, ncw * rl);
    const int hpx = hal_h * hal_w;
    ResP q;
    q.ci_p = (g.in_c + 31) / 32 * 32;
    q.hal_h = hal_h; q.hal_w = hal_w; q.kcc = kcc;
    q.lgv = log2i(pow2_ceil(kcc * 4));
    q.ltx = ltx; q.lty = lty; q.tiles = ltx * lty * g.batch;
    q.pitch = halo_pitch(g, hal_w);
    const size_t lds = std::max((size_t)hal_h * q.pitch * (kcc * 64 + 16), (size_t)(ksl - 1) * ncw * rl * 4 * 1024);
    const int nwv = ncw * ksl;
    // workgroups per compute unit: what registers and LDS allow, so that the memory round trips
    // of one workgroup's tile hide behind the others' reductions
    const int per_cu = std::max(1, 8 / nwv);
    const int slots = 256 * per_cu;
    dim3 grid((unsigned)std::min(q.tiles, std::max(1, slots / cbl)), cbl);
    const int nsw = ceil_div(g.kernel_h * g.kernel_w * kcc, ksl);
    note_kernel("conv_res_mfma_kernel");
    const int su = ceil_div(hpx, (nwv * WAVE) >> q.lgv);
#define DC_RES_S(RV, KV, NV, SV)                                                                             \
    conv_res_mfma_kernel<E, RV, KV, NV, SV><<<grid, nwv * WAVE, lds, s>>>(p, q, (const E *)in, (const E *)packed, \
                                                                          (const E *)bias, (E *)out, mask, out_mask)
#define DC_RES(RV, KV, NV)                                                                                   \
    do {                                                                                                     \
        if (su <= 4) DC_RES_S(RV, KV, NV, 4);                                                                \
        else if (su <= 8) DC_RES_S(RV, KV, NV, 8);                                                           \
        else DC_RES_S(RV, KV, NV, 12);                                                                       \
    } while (0)
#define DC_RES_N(RV, KV)                                                                                     \
    do {                                                                                                     \
        if (nsw <= 5) DC_RES(RV, KV, 5);                                                                     \
        else DC_RES(RV, KV, RES_MAX_STEPS);                                                                  \
    } while (0)
    if (rl == 1) DC_RES_N(1, 1);
    else if (ksl == 1) DC_RES_N(2, 1);
    else if (ksl == 2) DC_RES_N(2, 2);
    else DC_RES(2, 4, 5);
#undef DC_RES_N
#undef DC_RES
#undef DC_RES_S
    return hipGetLastError();
}

hipError_t launch_resident_conv(const dc_geometry &g, const ConvP &p, int hal_h, int hal_w, int ltx, int lty, int kcc,
                                int rl, int ksl, int ncw, const void *in, const void *packed, const void *bias,
                                void *out, const int32_t *mask, int32_t *out_mask, int dtype, hipStream_t s) {
    if (dtype == DC_BF16)
        return resident_t<bf16_t>(g, p, hal_h, hal_w, ltx, lty, kcc, rl, ksl, ncw, in, packed, bias, out, mask, out_mask, s);
    return resident_t<half_t>(g, p, hal_h, hal_w, ltx, lty, kcc, rl, ksl, ncw, in, packed, bias, out, mask, out_mask, s);
}

}  // namespace dc
