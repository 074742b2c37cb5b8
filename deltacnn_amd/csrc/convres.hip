// K x K delta convolution on the matrix cores for THIN layers on LARGE maps: the filter stays in
// registers and a workgroup walks over many output tiles.
//
// conv_lds_mfma_kernel (conv.hip) gives every 8x8 output tile a workgroup of its own, which
// streams its share of the filter from L2 -- for 64 -> 64 channels 73 KB per tile against 13 KB
// of input halo and 8 KB of output.  On a map of thousands of tiles that stream is most of the
// kernel's traffic and time.  Here a workgroup is launched once per compute-unit slot and loops
// over tiles (tile = blockIdx.x, blockIdx.x + gridDim.x, ...): the filter fragments of each
// wavefront's reduction steps (RES_STEPS steps x R channel tiles) are loaded before
// the loop and stay in registers, the step table is built once, and per tile only the mask words,
// the halo and the outputs move.  The loop is a two-stage pipeline with ONE barrier per tile:
// the mask words and halo rows of the NEXT tile are requested before the reduction of the current
// one (unconditionally, from clamped addresses, and selected by the mask afterwards) and staged
// into the second of two LDS halo buffers right after it; every wavefront dilates and compacts
// the tile's mask for itself; the partial sums of the reduction slices alternate between two
// buffers as well, so a wavefront that still finishes and stores tile i never holds up one that
// already contracts tile i + 1.  The slices of a channel group share the finishing of its tiles
// (each adds the partial sums of its share in ascending slice order, rounds and stores), and the
// walk from tile to tile is carried in (map, tile row, tile column) so that no tile costs a
// division; tiles whose halo lies inside the map skip the clamping of the row addresses.
//
// Everything else is the algorithm of conv_lds_mfma_kernel for a plain (not transposed)
// convolution whose input channels fit one LDS chunk: halo staged in LDS with inactive and
// out-of-bounds pixels as zeros, mask dilation and compaction of the tile's updated pixels by the
// first wavefront, wavefront = (channel group cw, reduction slice kz), slice kz taking steps
// kz, kz + KS, ... in ascending order, partial sums of the slices added in ascending slice order,
// one rounding after the bias.  An output element is accumulated by the same instruction sequence
// in both kernels, so they agree bit for bit.
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "epilogue.hpp"
#include "tile.hpp"

namespace dc {
namespace {

constexpr int RES_STEPS = 9;        // reduction steps per wavefront: their filter fragments stay in registers
constexpr int RES_MAX_HALO = 512;   // halo pixels (two tables in LDS)
constexpr int RES_MAX_TABLE = 96;   // reduction steps of a tile (taps x channel steps)

struct ResP {
    int ci_p, hal_h, hal_w, kcc, lgv;
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
    constexpr int TPW = R * NT / KS;  // output tiles of 16 x 16 a wavefront finishes
    static_assert(TPW * KS == R * NT, "the reduction slices of a channel group share its tiles evenly");
    // dynamic LDS: two halo buffers (tile i is contracted out of one while tile i + 1 is staged
    // into the other), then two buffers for the partial sums of the reduction slices
    extern __shared__ __align__(16) unsigned char s_dyn[];
    __shared__ int s_hpix[2][RES_MAX_HALO];
    __shared__ int2 s_step[RES_MAX_TABLE];
    __shared__ int s_wlist[8][TILE_PX];  // per wavefront: the tile's compacted updated pixels
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
    const int halo_bytes = hpx * row;
    unsigned char *s_part0 = s_dyn + 2 * halo_bytes;
    // every wavefront leaves the partial sums of the (KS - 1) * TPW tiles that other slices finish
    const int PART_BYTES = nw * (KS - 1) * TPW * WAVE * 16;
    auto tap_off = [&](int a, int b2) { return a * p.dh * hal_w + b2 * p.dw; };  // in halo pixels

    // step table: LDS byte offset of a step's input fragment relative to a pixel's halo origin
    // and its fragment offset in the packed filter; the same for every tile
    for (int j = tid; j < nsteps; j += nthr) {
        const int tap = j / ksteps, ks = j - tap * ksteps;
        const int ta = tap / p.Kw, tb = tap - ta * p.Kw;
        s_step[j] = int2{tap_off(ta, tb) * row + ks * 64, (tap * ksteps + ks) * 512};
    }
    __syncthreads();
    // the wavefront's filter fragments, resident for the whole kernel
    E8 a[NSW][R];
    int xoff[NSW];
#pragma unroll
    for (int i = 0; i < NSW; ++i) {
        const int2 e = s_step[min(i * KS + kz, nsteps - 1)];
        xoff[i] = __builtin_amdgcn_readfirstlane(e.x);  // the same in every lane of the wavefront
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
    int hrel[SU];              // ... and their pixel offset from the halo's first pixel in the map
#pragma unroll
    for (int u = 0; u < SU; ++u) {
        const int hp = min((tid >> q.lgv) + u * hstep, hpx - 1);
        const int hy = hp / hal_w;
        hyx[u] = (hy << 16) | (hp - hy * hal_w);
        hrel[u] = hy * p.Wi + (hp - hy * hal_w);
    }
    const int cst = min(sv * 8, p.Ci - 8);
    // A tile is (map b, tile row ty, tile column tx); the walk from tile to tile + gridDim.x is
    // carried in these coordinates, so that no tile costs a division.
    struct TilePos {
        int b, ty, tx;
    };
    const int gstep_b = (int)gridDim.x / tiles_per_map, gstep_r = (int)gridDim.x - gstep_b * tiles_per_map;
    const int gstep_y = gstep_r / q.ltx, gstep_x = gstep_r - gstep_y * q.ltx;
    auto advance = [&](TilePos t) {
        t.tx += gstep_x;
        t.ty += gstep_y;
        t.b += gstep_b;
        if (t.tx >= q.ltx) {
            t.tx -= q.ltx;
            ++t.ty;
        }
        if (t.ty >= q.lty) {
            t.ty -= q.lty;
            ++t.b;
        }
        return t;
    };
    auto request = [&](const TilePos &t) {
        const int iy0 = t.ty * TILE * p.sh - p.pt, ix0 = t.tx * TILE * p.sw - p.pl;
        const int32_t *mb = mask + (size_t)t.b * p.Hi * p.Wi;
        const E *inb = in + (size_t)t.b * p.Hi * p.Wi * p.Ci + cst;
        if (iy0 >= 0 && ix0 >= 0 && iy0 + hal_h <= p.Hi && ix0 + hal_w <= p.Wi) {  // uniform: nothing to clamp
            const int base = iy0 * p.Wi + ix0;
#pragma unroll
            for (int u = 0; u < SU; ++u) {
                const int px = base + hrel[u];
                hpixel[u] = px;
                word[u] = mb[px];
                val[u] = *reinterpret_cast<const E8 *>(inb + (unsigned)(px * p.Ci));
            }
        } else {
#pragma unroll
            for (int u = 0; u < SU; ++u) {
                const int iy = iy0 + (hyx[u] >> 16), ix = ix0 + (hyx[u] & 0xffff);
                const bool ok = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
                const int px = min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1);
                hpixel[u] = ok ? px : -1;
                word[u] = mb[px];
                val[u] = *reinterpret_cast<const E8 *>(inb + (unsigned)(px * p.Ci));
            }
        }
    };
    // what was requested goes into halo buffer `buf`: table entry (first lane of a pixel) and bytes
    auto stage = [&](int buf) {
        // What was requested has to have arrived here, for every lane: said once and without a
        // condition (s_waitcnt vmcnt(0)).  The stores below sit under per-lane tests, and a wait
        // that the compiler places inside them leaves it with a path on which the requests are
        // still in flight -- it then guards later writes of the same registers with waits that, at
        // run time, wait for the previous tile's output stores.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        const bool vok = sv < q.kcc * 4 && sv * 8 < p.Ci;
        unsigned char *halo = s_dyn + buf * halo_bytes;
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const int hp = (tid >> q.lgv) + u * hstep;
            const bool on = hpixel[u] >= 0 && word[u] != 0;
            if (hp < hpx) {
                if (sv == 0) s_hpix[buf][hp] = on ? hpixel[u] : -1;
                if (sv < q.kcc * 4)
                    *reinterpret_cast<E8 *>(halo + hp * row + sv * 16) = keep8(val[u], vok && on);
            }
        }
    };
    TilePos pos;
    {
        const int t0 = min((int)blockIdx.x, q.tiles - 1);
        pos.b = t0 / tiles_per_map;
        const int tr = t0 - pos.b * tiles_per_map;
        pos.ty = tr / q.ltx;
        pos.tx = tr - pos.ty * q.ltx;
    }
    TilePos nxt = advance(pos);
    if ((int)blockIdx.x < q.tiles) {
        request(pos);
        stage(0);
    }
    // Everything requested so far has arrived -- said explicitly (s_waitcnt vmcnt(0)): the compiler
    // cannot see it on every path into the loop and would otherwise wait for the resident filter
    // fragments in front of each matrix instruction of EVERY tile, where the count it waits on is
    // that of the next tile's rows, i.e. the reduction would stall until its prefetch has landed.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    // One barrier per tile.  Every wavefront dilates and compacts the tile's mask for itself (the
    // first one writes the output mask); the partial sums of tile i and the staged halo of tile
    // i + 1 become visible at the same barrier, behind which the finishing wavefronts store.
    int it = 0;
    for (int tile = blockIdx.x; tile < q.tiles; tile += gridDim.x, ++it, pos = nxt, nxt = advance(nxt)) {
        const int cur = it & 1;
        const int b = pos.b;
        const int ty0 = pos.ty * TILE, tx0 = pos.tx * TILE;
        // The next tile's mask words and rows travel while this tile is contracted.  Requested and
        // staged without a condition (behind the last tile: this tile once more, into the buffer
        // nobody reads): with the two under separate tests the compiler sees a path on which the
        // requests are never consumed and waits for ALL memory traffic -- the previous tile's
        // stores included -- at the head of every iteration.
        const bool has_next = tile + (int)gridDim.x < q.tiles;
        request(has_next ? nxt : pos);
        const unsigned char *halo = s_dyn + cur * halo_bytes;
        int n;
        {
            const int ly = lane >> 3, lx = lane & 7;
            const int oy = ty0 + ly, ox = tx0 + lx;
            const bool inside = oy < p.Ho && ox < p.Wo;
            bool upd = false;
            const int base = ly * p.sh * hal_w + lx * p.sw;
            if (p.Kh == 3 && p.Kw == 3) {  // the common window: nine independent reads
#pragma unroll
                for (int t = 0; t < 9; ++t) upd |= s_hpix[cur][base + tap_off(t / 3, t % 3)] >= 0;
            } else {
                for (int ta = 0; ta < p.Kh; ++ta)
                    for (int tb = 0; tb < p.Kw; ++tb) upd |= s_hpix[cur][base + tap_off(ta, tb)] >= 0;
            }
            upd = upd && inside;
            if (wv == 0 && inside && cb == 0) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = upd ? 1 : 0;
            const int rank = wave_rank(upd, n);
            if (upd) s_wlist[wv][rank] = lane;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        float4_t acc[R][NT];
        int loc[NT];
        if (n > 0) {  // the same for every wavefront
            const int n_tiles = (n + 15) >> 4;
            int hbase[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int slot = nt * 16 + l16;
                loc[nt] = slot < n ? s_wlist[wv][slot] : 0;
                hbase[nt] = ((loc[nt] >> 3) * p.sh * hal_w + (loc[nt] & 7) * p.sw) * row + kq * 16;
            }
            // (the tiles in use start from the first step's product; the others stay zero)
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[r][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
            // NSW steps for every wavefront (host: taps x channel steps == NSW * KS), one
            // branch-free block; the input fragments of a step are read from LDS while the matrix
            // instructions of the step before run
            auto reduce = [&](auto nta_tag) {
                constexpr int NTA = decltype(nta_tag)::value;
                E8 x[2][NTA];
#pragma unroll
                for (int nt = 0; nt < NTA; ++nt) x[0][nt] = *reinterpret_cast<const E8 *>(halo + hbase[nt] + xoff[0]);
#pragma unroll
                for (int i = 0; i < NSW; ++i) {
                    if (i + 1 < NSW) {
#pragma unroll
                        for (int nt = 0; nt < NTA; ++nt)
                            x[(i + 1) & 1][nt] = *reinterpret_cast<const E8 *>(halo + hbase[nt] + xoff[i + 1]);
                    }
                    // the reads above are issued before the matrix instructions below: left to
                    // itself the scheduler sinks every read to just before its use and waits for it
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
                        for (int r = 0; r < R; ++r)
                            acc[r][nt] = Elem16<E>::mfma(a[i][r], x[i & 1][nt], i == 0 ? float4_t{0.f, 0.f, 0.f, 0.f} : acc[r][nt]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            switch (n_tiles) {
                case 1: reduce(std::integral_constant<int, 1>{}); break;
                case 2: reduce(std::integral_constant<int, 2>{}); break;
                case 3: reduce(std::integral_constant<int, 3>{}); break;
                default: reduce(std::integral_constant<int, 4>{}); break;
            }
            if (KS > 1) {  // the tiles other slices finish: tile t of this wavefront in slot t (- TPW behind its own)
                float4_t *s_part = reinterpret_cast<float4_t *>(s_part0 + cur * PART_BYTES) + wv * (KS - 1) * TPW * WAVE;
#pragma unroll
                for (int t = 0; t < R * NT; ++t) {
                    if (t / TPW == kz) continue;  // uniform
                    s_part[(t < kz * TPW ? t : t - TPW) * WAVE + lane] = acc[t / NT][t % NT];
                }
            }
        }
        stage(cur ^ 1);
        __syncthreads();
        if (n == 0) continue;
        // The slices of a channel group share the finishing of its R * NT tiles: slice kz takes tiles
        // [kz * TPW, (kz + 1) * TPW), t = channel tile * NT + pixel tile, and adds the slices' partial
        // sums in ascending slice order (its own from registers).
        const float4_t *s_part = reinterpret_cast<const float4_t *>(s_part0 + cur * PART_BYTES);
        E *otile = out + (((size_t)b * p.Ho + ty0) * p.Wo + tx0) * p.Co;  // the tile's first output pixel
#pragma unroll
        for (int t = 0; t < R * NT; ++t) {
            if (KS > 1 && t / TPW != kz) continue;  // uniform
            const int r = t / NT, nt = t % NT;
            float4_t sum = acc[r][nt];
            if (KS > 1) {
#pragma unroll
                for (int z = 0; z < KS; ++z) {
                    // slice z's copy of tile t: in its wavefront's block, slot t (- TPW behind its own tiles)
                    float4_t term = acc[r][nt];
                    if (z != kz)  // uniform
                        term = s_part[(((z * ncw + cw) * (KS - 1) * TPW) + (t < z * TPW ? t : t - TPW)) * WAVE + lane];
                    sum = z == 0 ? term : sum + term;
                }
            }
            const int ct = (cb * ncw + cw) * R + r;
            if (ct >= co_tiles) continue;
            const int co = ct * 16 + kq * 4;  // lane holds channels co .. co + 3 of pixel (nt, l16)
            if (nt * 16 + l16 >= n) continue;
            E *o = otile + (unsigned)(((loc[nt] >> 3) * p.Wo + (loc[nt] & 7)) * p.Co + co);
            E4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = E(sum[i] + float(bv[r][i]));
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

}  // namespace

// Dynamic LDS of a launch: two halo buffers and two buffers of partial sums.
static size_t resident_lds(int hpx, int kcc, int rl, int ksl, int ncw) {
    return 2 * (size_t)hpx * (kcc * 64 + 16) + 2 * (size_t)(ksl - 1) * ncw * rl * 4 * 1024;
}

// Raises a kernel's dynamic LDS limit, once per kernel and device; a plain host call.
template <typename K>
static hipError_t allow_lds(K *kernel) {
    static std::atomic<uint64_t> done{0};  // one bit per device; devices past 63 ask every time
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 64 && ((done.load(std::memory_order_relaxed) >> dev) & 1ull)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 112 << 10);
    if (e == hipSuccess && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
    return e;
}

// Layers the resident-filter kernel takes, given the arrangement conv_lds_mfma_kernel would use
// (R channel tiles per wavefront, KS reduction slices, ncw channel groups, kcc channel steps per
// LDS chunk): 3 x 3 taps over two channel steps (33-64 input channels) with two channel tiles per
// wavefront and two reduction slices, LDS for two workgroups per compute unit, and enough tiles
// that walking over them pays.
bool resident_conv_eligible(const dc_geometry &g, int hal_h, int hal_w, int ltx, int lty, int kcc, int rl,
                            int ksl, int ncw) {
    const int ksteps = (g.in_c + 31) / 32;
    const int nsteps = g.kernel_h * g.kernel_w * ksteps;
    const int co_tiles = ceil_div(g.out_c, 16);
    const int cbl = ceil_div(co_tiles, ncw * rl);
    // Measured on 8 x 512 x 512 maps against conv_lds_mfma_kernel: 3 x 3 64 -> 64, whose filter takes
    // two channel steps, 399 -> 279 us at full density and 345 -> 224 us at 10 %; no gain or a loss
    // for a single channel step, whose filter of a few KB was never the cost (32 -> 64 stride 2:
    // 67 -> 70 us; 16 -> 16 on 544 x 960: 19.6 -> 22.8 us).
    if (kcc < 2) return false;
    // the arrangement that occurs in this range: two channel tiles per wavefront, two reduction
    // slices, nine steps each (3 x 3 taps x two channel steps); the reduction is one branch-free
    // block of exactly that many steps
    if (kcc != ksteps || nsteps > RES_MAX_TABLE || rl != 2 || ksl != 2 || nsteps != 2 * RES_STEPS) return false;
    const int hpx = hal_h * hal_w;
    if (hpx > RES_MAX_HALO) return false;
    // two workgroups per compute unit (with one, the form loses to the per-tile kernel: 64 -> 32 with
    // four reduction slices, whose partial sums take 48 KB, 397 us against 352 us)
    if (resident_lds(hpx, kcc, rl, ksl, ncw) > (72u << 10)) return false;
    const int hstep = (ncw * ksl * WAVE) >> log2i(pow2_ceil(kcc * 4));
    const int su = ceil_div(hpx, hstep);  // halo rows a lane keeps in flight
    if (su > 4) return false;  // (more halo rows in flight per lane would spill registers)
    // (offsets within one map of the batch are computed in 32 bits)
    if ((int64_t)g.in_h * g.in_w * g.in_c >= (1ll << 31) || (int64_t)g.out_h * g.out_w * g.out_c >= (1ll << 31)) return false;
    // (64 -> 64 on 136 x 240, 510 tiles per image: 10.4 against 9.9 us for one image, 15.3 against
    // 17.1 us for two, 24.4 against 30.7 us for four)
    return (int64_t)ltx * lty * g.batch * cbl >= 1024;
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
    const size_t lds = resident_lds(hpx, kcc, rl, ksl, ncw);
    const int nwv = ncw * ksl;
    // workgroups per compute unit: what registers and LDS allow, so that the memory round trips
    // of one workgroup's tile hide behind the others' reductions
    const int per_cu = std::max(1, 8 / nwv);
    const int slots = 256 * per_cu;
    dim3 grid((unsigned)std::min(q.tiles, std::max(1, slots / cbl)), cbl);
    note_kernel("conv_res_mfma_kernel");
    (void)rl;
    const hipError_t big = allow_lds(&conv_res_mfma_kernel<E, 2, 2, RES_STEPS, 4>);
    if (big != hipSuccess) return big;
    conv_res_mfma_kernel<E, 2, 2, RES_STEPS, 4><<<grid, nwv * WAVE, lds, s>>>(p, q, (const E *)in, (const E *)packed,
                                                                              (const E *)bias, (E *)out, mask, out_mask);
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
