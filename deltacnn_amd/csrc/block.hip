// One launch for the part of an inverted-residual network between two spatial convolutions:
//
//   A  depthwise 3x3 convolution + activation/truncation            (spatial: reads a 3x3 window)
//   B  1x1 projection (+ the block's residual sum, a DCAdd without activation)
//   C  1x1 expansion of the NEXT block + activation/truncation      (optional)
//
// B and C are pointwise, so a workgroup that owns 16 output pixels of A can carry them through
// all three stages without meeting another workgroup: the activated depthwise delta goes to the
// matrix cores through LDS and is never stored, and so does the block output on its way into
// the expansion.  Per frame this replaces three to four dependent launches by one, which is
// what bounds the frame time of a small-batch network.
//
// Arithmetic is that of the stand-alone kernels, operation for operation, so the results are
// identical to the separate calls bit for bit:
//   A  taps 0..8 in order, fp32 fma on zero-selected inputs, one rounding to fp16, then
//      T = trunc + v, S = T + prev, D = act(S) - act(prev), keep iff any |D| > thr
//      (conv_dw_kernel + act_trunc_pixel, truncation mode max)
//   B  v_mfma_f32_16x16x32_f16 over reduction steps of 32 hidden channels, taken by KW
//      interleaved slices (slice kw: steps kw, kw + KW, ...) whose partial sums are added in
//      ascending kw -- KW is what the stand-alone pointwise kernel picks for the same layer --
//      one rounding to fp16, then s = residual * wa, s = fma(conv, wb, s) (pw_mfma_kernel)
//   C  steps in ascending order in one accumulator, epilogue as in A (pw_act_mfma_kernel, or
//      pw_mfma_kernel followed by the activation kernel)
//
// Layout of a workgroup: G = 2^LG lanes per pixel in stage A (G >= hidden channels / 8 / ITERS),
// 16 pixels, hence NW = G / 4 wavefronts; in stages B and C the same wavefronts split the
// output channel tiles (and, in B, the reduction slices).
#include <atomic>

#include "epilogue.hpp"

namespace dc {
namespace {

struct BlockP {
    int B, Hi, Wi, Ho, Wo, sh, sw, pt, pl;
    int Ch;                           // hidden (depthwise) channels, a multiple of 8
    int Cp, cp_tiles, kp_steps, KWp;  // projection: channels, tiles of 16, reduction steps, slices
    int Ce, ce_tiles, ke_steps;       // expansion (Ce == 0: none)
    int px;                           // pixels per workgroup (block_eager_kernel)
    float thr_a, thr_c, wa, wb;
    const half_t *x;                  // depthwise input delta [B][Hi][Wi][Ch]
    const int32_t *xm;
    const half_t *wdw;                // depthwise filter [9][Ch]
    half_t *prev_a, *trunc_a;         // state of the depthwise layer's activation
    const half_t *wpj;                // packed projection filter
    const half_t *res;                // residual delta [P][Cp] or nullptr
    const int32_t *resm;
    half_t *out;                      // block output delta [P][Cp]
    int32_t *outm;
    const half_t *wex;                // packed expansion filter
    half_t *prev_c, *trunc_c;
    half_t *eout;                     // expansion output delta [P][Ce]
    int32_t *eoutm;
};

constexpr int PX = 16;      // pixels per workgroup
constexpr int RB = 4;       // projection tiles a wavefront accumulates per pass
constexpr int CTW_MAX = 6;  // expansion tiles per wavefront

// The 9 tap bits of pixel `pi` out of the 144 ballot bits (pixel-major, 9 per pixel).
__device__ __forceinline__ uint32_t tap_bits(const uint64_t (&bal)[3], int pi) {
    const int bit = pi * 9, w = bit >> 6, o = bit & 63;
    uint64_t v = (w == 0 ? bal[0] : w == 1 ? bal[1] : bal[2]) >> o;
    if (o > 55) v |= (w == 0 ? bal[1] : bal[2]) << (64 - o);  // w < 2 whenever o > 55 (bit <= 135)
    return uint32_t(v) & 0x1ffu;
}

template <int LG, int ITERS, int ACT>
__global__ void __launch_bounds__((PX << LG) < WAVE ? WAVE : (PX << LG))
block_dw_pw_kernel(BlockP p) {
    constexpr int G = 1 << LG;
    constexpr int NW = (PX * G) / WAVE;  // G >= 4
    constexpr int PPW = WAVE / G;        // pixels per wavefront in stage A
    constexpr int N = 8;                 // halves per 16-byte vector
    extern __shared__ __align__(16) unsigned char smem[];
    // LDS: flags | s_hid [16][Ch + 8] | s_out [16][Cp + 8] | s_red [NW][RB][64] float4 (KWp > 1)
    int *s_keep = reinterpret_cast<int *>(smem);             // [16] stage A keep flags
    int *s_stat = s_keep + PX;                               // [NW][16] stage C hits
    const int hid_ld = p.Ch + 8, out_ld = p.Cp + 8;
    half_t *s_hid = reinterpret_cast<half_t *>(smem + (PX + NW * PX) * sizeof(int));
    half_t *s_out = s_hid + PX * hid_ld;
    float4_t *s_red = reinterpret_cast<float4_t *>(s_out + PX * out_ld);

    const int wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int P = p.B * p.Ho * p.Wo;
    const int p0 = blockIdx.x * PX;

    // ---- masks: every wavefront derives the tap bits of all 16 pixels itself (3 loads per lane),
    // so the decision to leave needs no barrier
    uint64_t bal[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int e = lane + WAVE * i;
        const int pi = e / 9, t = e - pi * 9;
        bool m = false;
        const int po = p0 + pi;
        if (e < PX * 9 && po < P) {
            const int b = po / (p.Ho * p.Wo);
            const int r = po - b * p.Ho * p.Wo;
            const int oy = r / p.Wo, ox = r - oy * p.Wo;
            const int ky = t / 3, kx = t - ky * 3;
            const int iy = oy * p.sh - p.pt + ky, ix = ox * p.sw - p.pl + kx;
            if (iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi)
                m = p.xm[(size_t)b * p.Hi * p.Wi + iy * p.Wi + ix] != 0;
        }
        bal[i] = ballot(m);
    }
    int rword = 0;
    if (p.res != nullptr && lane < PX && p0 + lane < P) rword = p.resm[p0 + lane];
    const uint32_t br = uint32_t(ballot(rword != 0)) & 0xffffu;
    uint32_t bd = 0;  // pixels of the dilated mask
#pragma unroll
    for (int pi = 0; pi < PX; ++pi) bd |= (tap_bits(bal, pi) != 0 ? 1u : 0u) << pi;
    if ((bd | br) == 0) {  // nothing reaches this tile: all of its masks are 0
        if (wave == 0 && lane < PX && p0 + lane < P) {
            p.outm[p0 + lane] = 0;
            if (p.Ce > 0) p.eoutm[p0 + lane] = 0;
        }
        return;
    }

    // ---- stage A: depthwise 3x3 + activation/truncation, G lanes per pixel
    {
        const int pi = wave * PPW + lane / G, gl = lane & (G - 1);
        const int po = p0 + pi;
        const uint32_t taps = po < P ? tap_bits(bal, pi) : 0u;
        const bool active = taps != 0;
        const int pc = min(po, P - 1);
        const int b = pc / (p.Ho * p.Wo);
        const int r = pc - b * p.Ho * p.Wo;
        const int oy = r / p.Wo, ox = r - oy * p.Wo;
        const half_t *inb = p.x + (size_t)b * p.Hi * p.Wi * p.Ch;
        Vec<half_t, N> d[ITERS], tt[ITERS], ss[ITERS];
        bool hit = false;
        const half_t thr = half_t(p.thr_a);
        if (ballot(active) != 0) {  // wave-uniform: a wavefront without an updated pixel loads nothing
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = (it * G + gl) * N;
                const int cc = min(c, p.Ch - N);
                Vec<half_t, N> x[9], w[9];
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    const int ky = t / 3, kx = t - ky * 3;
                    const int iy = min(max(oy * p.sh - p.pt + ky, 0), p.Hi - 1);
                    const int ix = min(max(ox * p.sw - p.pl + kx, 0), p.Wi - 1);
                    x[t] = vload<half_t, N>(inb + (size_t)(iy * p.Wi + ix) * p.Ch + cc);
                    w[t] = vload<half_t, N>(p.wdw + (size_t)t * p.Ch + cc);
                }
                const Vec<half_t, N> q = vload<half_t, N>(p.prev_a + (size_t)pc * p.Ch + cc);
                const Vec<half_t, N> tr = vload<half_t, N>(p.trunc_a + (size_t)pc * p.Ch + cc);
                float acc[N];
#pragma unroll
                for (int j = 0; j < N; ++j) acc[j] = 0.f;
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    const Vec<half_t, N> xs = vkeep<half_t, N>(x[t], (taps >> t) & 1u);
#pragma unroll
                    for (int j = 0; j < N; ++j) acc[j] = __builtin_fmaf(float(xs.v[j]), float(w[t].v[j]), acc[j]);
                }
                if (active && c < p.Ch) {
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        const half_t v = half_t(acc[j]);
                        tt[it].v[j] = tr.v[j] + v;
                        ss[it].v[j] = tt[it].v[j] + q.v[j];
                        d[it].v[j] = act_apply<half_t>(ss[it].v[j], ACT) - act_apply<half_t>(q.v[j], ACT);
                        hit |= tabs(d[it].v[j]) > thr;
                    }
                }
            }
        }
        const bool keep = group_any(hit, G);
        if (active) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = (it * G + gl) * N;
                if (c < p.Ch) {
                    const size_t off = (size_t)po * p.Ch + c;
                    if (keep) {
                        Vec<half_t, N> z;
#pragma unroll
                        for (int j = 0; j < N; ++j) z.v[j] = half_t(0);
                        vstore<half_t, N>(p.prev_a + off, ss[it]);
                        vstore<half_t, N>(p.trunc_a + off, z);
                        vstore<half_t, N>(s_hid + pi * hid_ld + c, d[it]);
                    } else {
                        vstore<half_t, N>(p.trunc_a + off, tt[it]);
                    }
                }
            }
        }
        if (gl == 0) s_keep[pi] = (active && keep) ? 1 : 0;
    }
    __syncthreads();
    const uint32_t bk = uint32_t(ballot(lane < PX && s_keep[lane & (PX - 1)] != 0)) & 0xffffu;
    const uint32_t bo = bk | br;  // the block's output mask
    if (wave == 0 && lane < PX && p0 + lane < P) {
        p.outm[p0 + lane] = int((bo >> lane) & 1u);
        if (p.Ce > 0 && bo == 0) p.eoutm[p0 + lane] = 0;
    }
    if (bo == 0) return;  // every update of the tile was truncated away

    // ---- stage B: projection on the matrix cores (+ residual sum)
    {
        const int KW = p.KWp;
        const int kw = wave % KW, tg = wave / KW, ngroups = NW / KW;
        const half_t wa = half_t(p.wa), wb = half_t(p.wb);
        const bool on = (bk >> l16) & 1u, on_r = (br >> l16) & 1u;
        const size_t px = (size_t)(p0 + l16);
        // the SAME number of passes in every wavefront (there are barriers inside when KW > 1)
        for (int r0 = 0; r0 * ngroups < p.cp_tiles; r0 += RB) {
            float4_t acc[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
            if (bk != 0) {
                for (int s = kw; s < p.kp_steps; s += KW) {
                    const half8_t xf = *reinterpret_cast<const half8_t *>(
                        s_hid + l16 * hid_ld + min((s << 5) + kq * 8, p.Ch - 8));
                    half8_t a[RB];
#pragma unroll
                    for (int r = 0; r < RB; ++r) {
                        const int ct = min(tg + (r0 + r) * ngroups, p.cp_tiles - 1);
                        a[r] = *reinterpret_cast<const half8_t *>(p.wpj + ((size_t)ct * p.kp_steps + s) * 512 + lane * 8);
                    }
#pragma unroll
                    for (int r = 0; r < RB; ++r)
                        if (tg + (r0 + r) * ngroups < p.cp_tiles)  // wave-uniform
                            acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[r], xf, acc[r], 0, 0, 0);
                }
            }
            // finish: tile r of the pass by the wavefront with kw == r (KW == 1: every tile by its owner)
            if (KW > 1) {
#pragma unroll
                for (int r = 0; r < RB; ++r) s_red[(wave * RB + r) * WAVE + lane] = acc[r];
                __syncthreads();
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if (KW > 1 && kw != r) continue;                   // wave-uniform
                const int ct = tg + (r0 + r) * ngroups;
                if (ct >= p.cp_tiles) continue;                    // wave-uniform
                float4_t fin = acc[r];
                if (KW > 1) {
                    fin = s_red[((tg * KW) * RB + r) * WAVE + lane];
                    for (int q = 1; q < KW; ++q) fin += s_red[((tg * KW + q) * RB + r) * WAVE + lane];
                }
                const int co = ct * 16 + kq * 4;
                if (co >= p.Cp || !(on || on_r)) continue;
                half4_t o = half4_t{half_t(fin[0]), half_t(fin[1]), half_t(fin[2]), half_t(fin[3])};
                if (p.res != nullptr) {
                    half4_t rv = half4_t{0, 0, 0, 0};
                    if (on_r) rv = *reinterpret_cast<const half4_t *>(p.res + px * p.Cp + co);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        half_t sum = on_r ? half_t(rv[i] * wa) : half_t(0);
                        if (on) sum = fma_t(o[i], wb, sum);
                        o[i] = sum;
                    }
                }
                *reinterpret_cast<half4_t *>(p.out + px * p.Cp + co) = o;
                *reinterpret_cast<half4_t *>(s_out + l16 * out_ld + co) = o;
            }
            if (KW > 1) __syncthreads();  // s_red is reused by the next pass
        }
    }
    if (p.Ce == 0) return;
    __syncthreads();

    // ---- stage C: expansion on the matrix cores + activation/truncation
    {
        const bool on = (bo >> l16) & 1u;
        const size_t px = (size_t)min(p0 + l16, P - 1);
        half4_t q[CTW_MAX], tr[CTW_MAX];
        float4_t acc[CTW_MAX];
#pragma unroll
        for (int j = 0; j < CTW_MAX; ++j) {
            acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
            const int co = min(min(wave + j * NW, p.ce_tiles - 1) * 16 + kq * 4, p.Ce - 4);
            q[j] = *reinterpret_cast<const half4_t *>(p.prev_c + px * p.Ce + co);
            tr[j] = *reinterpret_cast<const half4_t *>(p.trunc_c + px * p.Ce + co);
        }
        for (int s = 0; s < p.ke_steps; ++s) {
            const half8_t xf = *reinterpret_cast<const half8_t *>(
                s_out + l16 * out_ld + min((s << 5) + kq * 8, p.Cp - 8));
            half8_t a[CTW_MAX];
#pragma unroll
            for (int j = 0; j < CTW_MAX; ++j) {
                const int ct = min(wave + j * NW, p.ce_tiles - 1);
                a[j] = *reinterpret_cast<const half8_t *>(p.wex + ((size_t)ct * p.ke_steps + s) * 512 + lane * 8);
            }
#pragma unroll
            for (int j = 0; j < CTW_MAX; ++j)
                if (wave + j * NW < p.ce_tiles)  // wave-uniform
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], xf, acc[j], 0, 0, 0);
        }
        const half_t thr = half_t(p.thr_c);
        half4_t v[CTW_MAX];
        bool hit = false;
#pragma unroll
        for (int j = 0; j < CTW_MAX; ++j) {
            const int ct = wave + j * NW;
            const bool live = ct < p.ce_tiles && ct * 16 + kq * 4 < p.Ce;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[j][i] = half_t(acc[j][i]);
                const half_t t = tr[j][i] + v[j][i];
                const half_t s = t + q[j][i];
                const half_t dd = act_apply<half_t>(s, ACT) - act_apply<half_t>(q[j][i], ACT);
                if (live && on) hit |= tabs(dd) > thr;
            }
        }
        const uint64_t hb = ballot(hit);
        if (kq == 0) s_stat[wave * PX + l16] = ((hb >> l16) & 0x0001000100010001ull) != 0 ? 1 : 0;
        __syncthreads();
        int tot = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) tot |= s_stat[w * PX + l16];
        const bool keep = tot != 0;
        if (wave == 0 && kq == 0 && p0 + l16 < P) p.eoutm[p0 + l16] = (on && keep) ? 1 : 0;
        if (!on) return;
#pragma unroll
        for (int j = 0; j < CTW_MAX; ++j) {
            const int ct = wave + j * NW;
            if (ct >= p.ce_tiles) break;  // wave-uniform
            const int co = ct * 16 + kq * 4;
            if (co >= p.Ce) continue;
            const size_t off = px * p.Ce + co;
            half4_t t, s, dd;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                t[i] = tr[j][i] + v[j][i];
                s[i] = t[i] + q[j][i];
                dd[i] = act_apply<half_t>(s[i], ACT) - act_apply<half_t>(q[j][i], ACT);
            }
            if (keep) {
                *reinterpret_cast<half4_t *>(p.prev_c + off) = s;
                *reinterpret_cast<half4_t *>(p.eout + off) = dd;
                *reinterpret_cast<half4_t *>(p.trunc_c + off) = half4_t{0, 0, 0, 0};
            } else {
                *reinterpret_cast<half4_t *>(p.trunc_c + off) = t;
            }
        }
    }
}

// The same block for layers whose filters are a few KB (the large maps at the front of a network):
// EVERYTHING whose address depends on coordinates only -- mask words, the 3x3 window of every
// pixel, the depthwise filter, the depthwise layer's cached state, the residual and ALL filter
// fragments of both pointwise convolutions -- is requested before the first value is waited for,
// so the kernel is one memory round trip, three barriers and the stores; what was loaded for an
// inactive tile is dropped.  The expansion's cached state alone is requested behind the mask
// test, by workgroups that have an update: it is needed two barriers later, so the second
// round trip hides behind the first two stages, and idle workgroups do not fetch it (measured
// on the MobileNetV2 frame, builds alternating on one device: 5667 against 5642 frames/s).
// Arithmetic and summation order are those of block_dw_pw_kernel.
// Requires: one vector per lane in stage A (Ch <= 8 G), G <= 32 (at most 8 wavefronts, so a
// wavefront may hold 256 registers), no reduction split, at most KPS_E projection steps and one
// projection tile per wavefront, one expansion step (Cp <= 32), at most CTW_E expansion tiles
// per wavefront.
constexpr int KPS_E = 6, CTW_E = 6;

template <int LG, int ACT>
__global__ void __launch_bounds__((PX << LG) < WAVE ? WAVE : (PX << LG))
block_eager_kernel(BlockP p) {
    constexpr int G = 1 << LG;
    constexpr int NW = (PX * G) / WAVE;
    constexpr int PPW = WAVE / G;
    constexpr int N = 8;
    extern __shared__ __align__(16) unsigned char smem[];
    int *s_keep = reinterpret_cast<int *>(smem);
    int *s_stat = s_keep + PX;
    const int hid_ld = p.Ch + 8, out_ld = p.Cp + 8;
    half_t *s_hid = reinterpret_cast<half_t *>(smem + (PX + NW * PX) * sizeof(int));
    half_t *s_out = s_hid + PX * hid_ld;

    const int wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    // A workgroup takes p.px (<= 16) consecutive pixels: fewer than 16 on small maps, so that the
    // launch has enough workgroups to draw on every compute unit's memory path (the pixel slots
    // past p.px shadow the last pixel and store nothing).  P = one past the workgroup's last pixel.
    const int p0 = blockIdx.x * p.px;
    const int P = min(p.B * p.Ho * p.Wo, p0 + p.px);

    // ---- every request of the kernel
    bool mbit[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int e = lane + WAVE * i;
        const int pi = e / 9, t = e - pi * 9;
        const int po = min(p0 + pi, P - 1);
        const int b = po / (p.Ho * p.Wo);
        const int r = po - b * p.Ho * p.Wo;
        const int oy = r / p.Wo, ox = r - oy * p.Wo;
        const int ky = t / 3, kx = t - ky * 3;
        const int iy = oy * p.sh - p.pt + ky, ix = ox * p.sw - p.pl + kx;
        const bool inside = e < PX * 9 && p0 + pi < P && iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
        const int word = p.xm[(size_t)b * p.Hi * p.Wi + min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1)];
        mbit[i] = inside && word != 0;
    }
    int rword = 0;
    if (p.res != nullptr) rword = p.resm[min(p0 + l16, P - 1)];
    // stage A operands of this lane's (pixel, channel vector)
    const int pi = wave * PPW + lane / G, gl = lane & (G - 1);
    const int po = p0 + pi;
    const int pc = min(po, P - 1);
    const int c = gl * N;
    const int cc = min(c, p.Ch - N);
    // (Requests are made only by lanes and wavefronts that will use what they ask for -- the pixel
    // slots of this workgroup that hold a pixel, the wavefronts that own a projection or expansion
    // tile, the reduction steps that exist: a compute unit issues 64 bytes of requests per clock,
    // and the rows, filters and fragments of a workgroup are 60-250 KB of them.)
    const half8_t zero8 = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    half8_t x[9], w[9], qa = zero8, tra = zero8;
#pragma unroll
    for (int t = 0; t < 9; ++t) x[t] = w[t] = zero8;
    if (po < P && c < p.Ch) {
        const int b = pc / (p.Ho * p.Wo);
        const int r = pc - b * p.Ho * p.Wo;
        const int oy = r / p.Wo, ox = r - oy * p.Wo;
        const half_t *inb = p.x + (size_t)b * p.Hi * p.Wi * p.Ch;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int ky = t / 3, kx = t - ky * 3;
            const int iy = min(max(oy * p.sh - p.pt + ky, 0), p.Hi - 1);
            const int ix = min(max(ox * p.sw - p.pl + kx, 0), p.Wi - 1);
            x[t] = *reinterpret_cast<const half8_t *>(inb + (size_t)(iy * p.Wi + ix) * p.Ch + cc);
            w[t] = *reinterpret_cast<const half8_t *>(p.wdw + (size_t)t * p.Ch + cc);
        }
        qa = *reinterpret_cast<const half8_t *>(p.prev_a + (size_t)pc * p.Ch + cc);
        tra = *reinterpret_cast<const half8_t *>(p.trunc_a + (size_t)pc * p.Ch + cc);
    }
    // stage B: the projection tile of this wavefront (wavefronts past the last tile shadow it)
    const int ct_b = min(wave, p.cp_tiles - 1);
    const size_t pxl = (size_t)min(p0 + l16, P - 1);
    half8_t afr[KPS_E];
#pragma unroll
    for (int s = 0; s < KPS_E; ++s) {
        afr[s] = zero8;
        if (wave < p.cp_tiles && s < p.kp_steps)  // uniform
            afr[s] = *reinterpret_cast<const half8_t *>(p.wpj + ((size_t)ct_b * p.kp_steps + s) * 512 + lane * 8);
    }
    const int co_b = min(ct_b * 16 + kq * 4, p.Cp - 4);
    half4_t rv = half4_t{0, 0, 0, 0};
    if (p.res != nullptr && wave < p.cp_tiles) rv = *reinterpret_cast<const half4_t *>(p.res + pxl * p.Cp + co_b);
    // stage C: filter fragments (one step) and cached state of this wavefront's tiles
    half8_t efr[CTW_E];
    half4_t qc[CTW_E], trc[CTW_E];
    if (p.Ce > 0) {
#pragma unroll
        for (int j = 0; j < CTW_E; ++j) {
            efr[j] = zero8;
            if (wave + j * NW < p.ce_tiles)  // uniform
                efr[j] = *reinterpret_cast<const half8_t *>(p.wex + (size_t)(wave + j * NW) * 512 + lane * 8);
        }
    }
    // all of the above is in flight before anything is waited for
#pragma unroll
    for (int t = 0; t < 9; ++t) {
        DC_PIN(x[t]);
        DC_PIN(w[t]);
    }
    DC_PIN(qa);
    DC_PIN(tra);
#pragma unroll
    for (int s = 0; s < KPS_E; ++s) DC_PIN(afr[s]);
    DC_PIN(rv);
    if (p.Ce > 0) {
#pragma unroll
        for (int j = 0; j < CTW_E; ++j) {
            DC_PIN(efr[j]);
        }
    }

    uint64_t bal[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) bal[i] = ballot(mbit[i]);
    const uint32_t br = uint32_t(ballot(lane < PX && p0 + lane < P && rword != 0)) & 0xffffu;
    uint32_t bd = 0;
#pragma unroll
    for (int q = 0; q < PX; ++q) bd |= (tap_bits(bal, q) != 0 ? 1u : 0u) << q;
    if ((bd | br) == 0) {
        if (wave == 0 && lane < PX && p0 + lane < P) {
            p.outm[p0 + lane] = 0;
            if (p.Ce > 0) p.eoutm[p0 + lane] = 0;
        }
        return;
    }
    // the expansion's cached state, for workgroups with something to do: it is needed two
    // barriers from here
    if (p.Ce > 0) {
#pragma unroll
        for (int j = 0; j < CTW_E; ++j) {
            qc[j] = trc[j] = half4_t{0, 0, 0, 0};
            const int ct = wave + j * NW;
            if (ct >= p.ce_tiles) continue;  // uniform
            const int co = min(ct * 16 + kq * 4, p.Ce - 4);
            qc[j] = *reinterpret_cast<const half4_t *>(p.prev_c + pxl * p.Ce + co);
            trc[j] = *reinterpret_cast<const half4_t *>(p.trunc_c + pxl * p.Ce + co);
        }
    }

    // ---- stage A
    {
        const uint32_t taps = po < P ? tap_bits(bal, pi) : 0u;
        const bool active = taps != 0;
        float acc[N];
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] = 0.f;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const half8_t xs = keep8(x[t], (taps >> t) & 1u);
#pragma unroll
            for (int j = 0; j < N; ++j) acc[j] = __builtin_fmaf(float(xs[j]), float(w[t][j]), acc[j]);
        }
        half8_t d, tt, ss;
        bool hit = false;
        const half_t thr = half_t(p.thr_a);
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const half_t v = half_t(acc[j]);
            tt[j] = tra[j] + v;
            ss[j] = tt[j] + qa[j];
            d[j] = act_apply<half_t>(ss[j], ACT) - act_apply<half_t>(qa[j], ACT);
            if (active && c < p.Ch) hit |= tabs(d[j]) > thr;
        }
        const bool keep = group_any(hit, G);
        if (active && c < p.Ch) {
            const size_t off = (size_t)po * p.Ch + c;
            if (keep) {
                *reinterpret_cast<half8_t *>(p.prev_a + off) = ss;
                *reinterpret_cast<half8_t *>(p.trunc_a + off) = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                *reinterpret_cast<half8_t *>(s_hid + pi * hid_ld + c) = d;
            } else {
                *reinterpret_cast<half8_t *>(p.trunc_a + off) = tt;
            }
        }
        if (gl == 0) s_keep[pi] = (active && keep) ? 1 : 0;
    }
    __syncthreads();
    const uint32_t bk = uint32_t(ballot(lane < PX && s_keep[lane & (PX - 1)] != 0)) & 0xffffu;
    const uint32_t bo = bk | br;
    if (wave == 0 && lane < PX && p0 + lane < P) {
        p.outm[p0 + lane] = int((bo >> lane) & 1u);
        if (p.Ce > 0 && bo == 0) p.eoutm[p0 + lane] = 0;
    }
    if (bo == 0) return;

    // ---- stage B: one tile per wavefront, steps in ascending order
    if (wave < p.cp_tiles) {  // wave-uniform
        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
        if (bk != 0) {
#pragma unroll
            for (int s = 0; s < KPS_E; ++s) {
                if (s < p.kp_steps) {  // uniform
                    const half8_t xf = *reinterpret_cast<const half8_t *>(
                        s_hid + l16 * hid_ld + min((s << 5) + kq * 8, p.Ch - 8));
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(afr[s], xf, acc, 0, 0, 0);
                }
            }
        }
        const bool on = (bk >> l16) & 1u, on_r = (br >> l16) & 1u;
        const int co = wave * 16 + kq * 4;
        if (co < p.Cp && (on || on_r)) {
            half4_t o = half4_t{half_t(acc[0]), half_t(acc[1]), half_t(acc[2]), half_t(acc[3])};
            if (p.res != nullptr) {
                const half_t wa = half_t(p.wa), wb = half_t(p.wb);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    half_t sum = on_r ? half_t(rv[i] * wa) : half_t(0);
                    if (on) sum = fma_t(o[i], wb, sum);
                    o[i] = sum;
                }
            }
            *reinterpret_cast<half4_t *>(p.out + (size_t)(p0 + l16) * p.Cp + co) = o;
            *reinterpret_cast<half4_t *>(s_out + l16 * out_ld + co) = o;
        }
    }
    if (p.Ce == 0) return;
    __syncthreads();

    // ---- stage C: one reduction step
    {
        const bool on = (bo >> l16) & 1u;
        const half8_t xf = *reinterpret_cast<const half8_t *>(s_out + l16 * out_ld + min(kq * 8, p.Cp - 8));
        const half_t thr = half_t(p.thr_c);
        half4_t v[CTW_E];
        bool hit = false;
#pragma unroll
        for (int j = 0; j < CTW_E; ++j) {
            const int ct = wave + j * NW;
            float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
            if (ct < p.ce_tiles) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(efr[j], xf, acc, 0, 0, 0);  // uniform
            const bool live = ct < p.ce_tiles && ct * 16 + kq * 4 < p.Ce;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[j][i] = half_t(acc[i]);
                const half_t t = trc[j][i] + v[j][i];
                const half_t s = t + qc[j][i];
                const half_t dd = act_apply<half_t>(s, ACT) - act_apply<half_t>(qc[j][i], ACT);
                if (live && on) hit |= tabs(dd) > thr;
            }
        }
        const uint64_t hb = ballot(hit);
        if (kq == 0) s_stat[wave * PX + l16] = ((hb >> l16) & 0x0001000100010001ull) != 0 ? 1 : 0;
        __syncthreads();
        int tot = 0;
#pragma unroll
        for (int q = 0; q < NW; ++q) tot |= s_stat[q * PX + l16];
        const bool keep = tot != 0;
        if (wave == 0 && kq == 0 && p0 + l16 < P) p.eoutm[p0 + l16] = (on && keep) ? 1 : 0;
        if (!on) return;
#pragma unroll
        for (int j = 0; j < CTW_E; ++j) {
            const int ct = wave + j * NW;
            if (ct >= p.ce_tiles) break;  // wave-uniform
            const int co = ct * 16 + kq * 4;
            if (co >= p.Ce) continue;
            const size_t off = pxl * p.Ce + co;
            half4_t t, s, dd;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                t[i] = trc[j][i] + v[j][i];
                s[i] = t[i] + qc[j][i];
                dd[i] = act_apply<half_t>(s[i], ACT) - act_apply<half_t>(qc[j][i], ACT);
            }
            if (keep) {
                *reinterpret_cast<half4_t *>(p.prev_c + off) = s;
                *reinterpret_cast<half4_t *>(p.eout + off) = dd;
                *reinterpret_cast<half4_t *>(p.trunc_c + off) = half4_t{0, 0, 0, 0};
            } else {
                *reinterpret_cast<half4_t *>(p.trunc_c + off) = t;
            }
        }
    }
}

// Raises a kernel's dynamic LDS limit to 128 KB, once per kernel and device (the attribute belongs
// to the device's copy of the function); a plain host call, nothing is put on a stream.
template <typename K>
hipError_t allow_lds(K *kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return hipSuccess;
    static std::atomic<uint64_t> done{0};  // one bit per device; devices past 63 ask every time
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 64 && ((done.load(std::memory_order_relaxed) >> dev) & 1ull)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            128 * 1024);
    if (e == hipSuccess && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
    return e;
}

}  // namespace

// Shapes the fused block kernel takes; everything else is reported as unsupported before any
// launch, and the caller issues the separate calls.
const char *block_unsupported(const dc_geometry &g, const dc_block_args &b, int dtype) {
    if (dtype != DC_F16) return "fp16 only";
    if (g.groups != g.in_c || g.in_c != g.out_c) return "the first convolution must be depthwise";
    if (g.kernel_h != 3 || g.kernel_w != 3 || g.dilation_h != 1 || g.dilation_w != 1) return "3x3 window, dilation 1";
    if (g.in_c % 8 != 0 || g.in_c > 1024) return "hidden channels: a multiple of 8, at most 1024";
    if (b.project_channels % 8 != 0 || b.project_channels < 8 || b.project_channels > 512)
        return "projection channels: a multiple of 8 in 8..512";
    if (b.dw_truncation_mode != DC_TRUNC_MAX) return "truncation mode max only";
    const int act = b.dw_activation;
    if (act != DC_ACT_RELU && act != DC_ACT_RELU6 && act != DC_ACT_LEAKY) return "activation relu, relu6 or leaky";
    if (b.expand_channels > 0) {
        if (b.expand_activation != act || b.expand_truncation_mode != DC_TRUNC_MAX)
            return "both activations must be the same, truncation mode max";
        if (b.expand_channels % 4 != 0) return "expansion channels: a multiple of 4";
    }
    return nullptr;
}

hipError_t launch_block(const dc_geometry &g, const dc_block_args &b, hipStream_t s, const char **why) {
    BlockP p;
    p.B = g.batch; p.Hi = g.in_h; p.Wi = g.in_w; p.Ho = g.out_h; p.Wo = g.out_w;
    p.sh = g.stride_h; p.sw = g.stride_w; p.pt = g.pad_top; p.pl = g.pad_left;
    p.Ch = g.in_c;
    const int P = g.batch * g.out_h * g.out_w;
    p.Cp = b.project_channels; p.cp_tiles = ceil_div(p.Cp, 16); p.kp_steps = ceil_div(p.Ch, 32);
    p.KWp = pointwise_reduction_slices(P, p.Ch, p.Cp);
    p.px = PX;
    p.Ce = b.expand_channels; p.ce_tiles = ceil_div(p.Ce, 16); p.ke_steps = ceil_div(p.Cp, 32);
    p.thr_a = b.dw_threshold; p.thr_c = b.expand_threshold; p.wa = b.weight_residual; p.wb = b.weight_conv;
    p.x = (const half_t *)b.input; p.xm = b.mask; p.wdw = (const half_t *)b.dw_filter;
    p.prev_a = (half_t *)b.dw_prev_out; p.trunc_a = (half_t *)b.dw_truncated;
    p.wpj = (const half_t *)b.project_packed_filter;
    p.res = (const half_t *)b.residual; p.resm = b.residual_mask;
    p.out = (half_t *)b.out; p.outm = b.out_mask;
    p.wex = (const half_t *)b.expand_packed_filter;
    p.prev_c = (half_t *)b.expand_prev_out; p.trunc_c = (half_t *)b.expand_truncated;
    p.eout = (half_t *)b.expand_out; p.eoutm = b.expand_out_mask;

    // lanes per pixel of the depthwise stage: one or two 16-byte vectors per lane
    const int nvec = p.Ch / 8;
    int lg = 2;
    while ((1 << lg) < nvec && lg < 6) ++lg;
    const int iters = ceil_div(nvec, 1 << lg);
    const int nw = (PX << lg) / WAVE;
    *why = nullptr;
    if (iters > 2) { *why = "more than 1024 hidden channels"; return hipSuccess; }
    if (p.KWp > 1 && (nw % p.KWp != 0 || p.KWp < RB)) { *why = "reduction split does not fit the workgroup"; return hipSuccess; }
    if (p.Ce > 0) {
        if (pointwise_reduction_slices(P, p.Cp, p.Ce) != 1) { *why = "the expansion's reduction would be split"; return hipSuccess; }
        if (ceil_div(p.ce_tiles, nw) > CTW_MAX) { *why = "too many expansion channels for this hidden width"; return hipSuccess; }
    }
    size_t lds = (PX + nw * PX) * sizeof(int) + (size_t)PX * (p.Ch + 8) * 2 + (size_t)PX * (p.Cp + 8) * 2;
    lds = (lds + 15) / 16 * 16;
    if (p.KWp > 1) lds += (size_t)nw * RB * WAVE * sizeof(float4_t);
    if (lds > 128 * 1024) { *why = "LDS"; return hipSuccess; }
    const dim3 grid(ceil_div(P, PX));
    // small filters and at most 8 wavefronts: the one-round-trip form
    const bool eager = iters == 1 && lg <= 5 && p.KWp == 1 && p.kp_steps <= KPS_E && p.cp_tiles <= nw &&
                       (p.Ce == 0 || (p.ke_steps == 1 && p.ce_tiles <= CTW_E * nw)) && !(b.flags & DC_BLOCK_LATE_LOADS);
    if (eager) {
        // 16 pixels per workgroup from 128 workgroups on, else 4 (measured on 28x28 maps of 144-192
        // channels: 8.2-8.9 us against 9.8-10.7 with 16; on 56x56 the smaller tile loses, every
        // workgroup re-reads both filters)
        p.px = P >= 2048 ? 16 : 4;
        const dim3 grid(ceil_div(P, p.px));
        note_kernel("block_eager_kernel");
#define DC_BLOCK_E(LGv, A)                                                                   \
    do {                                                                                     \
        block_eager_kernel<LGv, A><<<grid, (PX << LGv) < WAVE ? WAVE : (PX << LGv), lds, s>>>(p); \
        return hipGetLastError();                                                            \
    } while (0)
#define DC_BLOCK_EA(LGv)                                                                     \
    switch (b.dw_activation) {                                                               \
        case DC_ACT_RELU: DC_BLOCK_E(LGv, DC_ACT_RELU);                                      \
        case DC_ACT_RELU6: DC_BLOCK_E(LGv, DC_ACT_RELU6);                                    \
        default: DC_BLOCK_E(LGv, DC_ACT_LEAKY);                                              \
    }
        if (lg == 2) DC_BLOCK_EA(2)
        if (lg == 3) DC_BLOCK_EA(3)
        if (lg == 4) DC_BLOCK_EA(4)
        DC_BLOCK_EA(5)
#undef DC_BLOCK_EA
#undef DC_BLOCK_E
    }
    note_kernel("block_dw_pw_kernel");
#define DC_BLOCK_GO(LGv, IT, A)                                                              \
    do {                                                                                     \
        hipError_t e = allow_lds(block_dw_pw_kernel<LGv, IT, A>, lds);                       \
        if (e != hipSuccess) return e;                                                       \
        block_dw_pw_kernel<LGv, IT, A><<<grid, (PX << LGv) < WAVE ? WAVE : (PX << LGv), lds, s>>>(p); \
        return hipGetLastError();                                                            \
    } while (0)
#define DC_BLOCK_ACT(LGv, IT)                                                                \
    switch (b.dw_activation) {                                                               \
        case DC_ACT_RELU: DC_BLOCK_GO(LGv, IT, DC_ACT_RELU);                                 \
        case DC_ACT_RELU6: DC_BLOCK_GO(LGv, IT, DC_ACT_RELU6);                               \
        default: DC_BLOCK_GO(LGv, IT, DC_ACT_LEAKY);                                         \
    }
    if (lg == 2) DC_BLOCK_ACT(2, 1)
    if (lg == 3) DC_BLOCK_ACT(3, 1)
    if (lg == 4) DC_BLOCK_ACT(4, 1)
    if (lg == 5) DC_BLOCK_ACT(5, 1)
    if (iters == 1) DC_BLOCK_ACT(6, 1)
    DC_BLOCK_ACT(6, 2)
#undef DC_BLOCK_ACT
#undef DC_BLOCK_GO
    return hipErrorInvalidValue;
}

}  // namespace dc
