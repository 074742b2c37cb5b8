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
// (fragment order, one contiguous KB per channel tile and step), columns = 16 pixels (NHWC rows), fp32 accumulate, reduction in
// steps of 32 input channels taken in ascending order (both kernels below and the generic
// kernel accumulate a given output element with the same instruction sequence, so they agree
// bit for bit).
//
// pw_mfma_kernel      convolution only (optionally + residual add); the arrangement of a
//                     workgroup's wavefronts over reduction slices, channel tiles and pixel
//                     tiles is a template parameter set chosen per layer by the host
// pw_act_mfma_kernel  convolution + activation/truncation in one launch: a workgroup owns ALL
//                     output channels of its 16 pixels, so it can take the per-pixel keep/drop
//                     decision itself; the convolution output never travels through memory.
//                     Used while the filter fragments of a wavefront fit in registers (up to
//                     8 channel tiles x 5 reduction steps); larger layers keep the two-launch
//                     form, whose channel split over many workgroups streams big filters fast
#include "epilogue.hpp"

namespace dc {
namespace {

struct PwP {
    int P, Ci, Co, ci_p, co_tiles;
    // XCD-aware launch (xcd != 0): the grid is one-dimensional, nx * round_up(ny, 8) workgroups.
    // The hardware deals workgroups to the 8 XCDs round-robin by linear id, each XCD has its own
    // L2; workgroup L takes channel group (L % 8) + 8 * ((L / 8) / nx) and pixel tile
    // (L / 8) % nx, so all pixel tiles of a channel group run on ONE XCD and its filter
    // fragments are fetched into one L2 instead of up to eight.
    int xcd, nx, ny;
};

// ADD fuses the residual sum of a DCAdd layer behind the convolution: with a = residual delta
// (mask Ma) and b = convolution output rounded to fp16 (mask Mb = input mask),
// out = fma(b, wb, a * wa) on pixels of Ma | Mb, each term present only where its mask is set --
// the same operations, in the same order and precision, as the stand-alone add kernel.
template <typename E>
struct ResP {
    const E *res;  // MODE 3: the layer's truncated values (read; T is written back through `tmp`)
    const int32_t *mask;
    float wa, wb;
    E *prev;  // MODE 2: the sum is accumulated here and its activated difference is emitted; MODE 3: read only
    int act;
    E *tmp = nullptr;  // MODE 3: the layer's truncated values again, which receive T = truncated + v
};

// MODE 4: the input is the concatenation, along the channels, of up to four delta tensors with
// masks of their own (a DCConcatenate chain in front of the convolution, which then never
// runs): reduction step s belongs to the tensor whose step range holds it, a pixel's fragment
// counts only where that tensor's mask is set, and the output mask is the union -- the products
// a concatenated tensor's zero-filled halves would add are exact zeros, so the result equals the
// convolution of the concatenation bit for bit.  Unused entries repeat entry 0 with a step range
// that is never reached.
constexpr int PW_MAX_SEGS = 4;
template <typename E>
struct PwSegs {
    const E *in[PW_MAX_SEGS];
    const int32_t *mask[PW_MAX_SEGS];
    int C[PW_MAX_SEGS];          // channels, multiples of 32
    int step0[PW_MAX_SEGS];      // first reduction step
    int n;
};

// A workgroup takes 64 consecutive pixels (4 pixel tiles of 16) x CBW * R channel tiles of 16.
// Its KW * CBW * NBW wavefronts are arranged as
//   KW  slices of the reduction (wavefront kw takes steps kw, kw + KW, ...; the partial sums
//       meet in LDS and are added in ascending kw, so the result does not depend on timing),
//   CBW groups of R channel tiles,
//   NBW groups of NTW pixel tiles (NBW * NTW == 4),
// so a wavefront accumulates R x NTW tiles and needs R filter + NTW input fragments per
// reduction step.  The host picks the arrangement per layer: many pixels and few channels
// favour NBW > 1, few pixels and a long reduction favour KW > 1 with R > 1 (the input
// fragments are then shared by R channel tiles instead of being fetched again by other
// workgroups).  S = reduction steps per memory round trip: all fragment loads of S steps are in
// flight together.
// MODE: 0 convolution only, 1 fused sum, 2 fused sum with the DCAdd layer's activation,
// 3 the layer's own activation left OPEN: with v the convolution result, T = truncated + v,
// S = T + prev, D = act(S) - act(prev) (one rounding each, the sequence of act_trunc_pixel), the
// kernel emits D as its output, replaces the layer's truncated values by T for every updated pixel
// (what they have to hold if the pixel is dropped) and leaves the accumulated values alone; whether a pixel is kept -- any |D| of its channels above the threshold -- is
// decided by the depthwise kernel that consumes D (conv_dw_kernel<FIN>), which also commits
// the state.  A workgroup holds a slice of a pixel's channels, so it cannot decide itself.
// ACTC >= 0: the activation of MODE 2 / 3 as a compile-time constant (a run-time id costs a chain
// of scalar branches per element, half a microsecond in a kernel of this size); -1: rp.act.
// (bx, by): the workgroup's pixel group and channel group; s_red: KW * CBW * NBW * R * NTW * WAVE
// partial sums in LDS (KW > 1).
template <typename E, int KW, int CBW, int NBW, int R, int NTW, int S, int MODE, bool EAGER, int ACTC = -1>
__device__ __forceinline__ void
pw_mfma_body(const PwP &p, const E *__restrict__ in, const E *__restrict__ wp,
             const E *__restrict__ bias, E *__restrict__ out,
             const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, const ResP<E> &rp,
             int bx, int by, float4_t *s_red, E *s_open = nullptr, const PwSegs<E> *sgp = nullptr) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    static_assert(NBW * NTW <= 4, "a workgroup covers at most 64 pixels");
    constexpr bool ADD = MODE == 1 || MODE == 2, ADDACT = MODE == 2, OPEN = MODE == 3, SEG = MODE == 4;
    constexpr int NW = KW * CBW * NBW, TILES = R * NTW, FT = (TILES + KW - 1) / KW;
    constexpr int PXW = NBW * NTW * 16;  // pixels per workgroup
    const int wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int kw = wave % KW, tw = wave / KW, cw = tw % CBW, nw = tw / CBW;
    const int ksteps = p.ci_p >> 5;
    const int pbase = bx * PXW;

    // the mask words of the workgroup's pixels, one per lane, together with the first chunk
    // of filter fragments (which do not depend on the masks)
    const int mp = pbase + lane;
    const bool mine = lane < PXW && mp < p.P;
    int mword = 0, sword[PW_MAX_SEGS] = {0, 0, 0, 0};
    if (SEG) {
#pragma unroll
        for (int g = 0; g < PW_MAX_SEGS; ++g) sword[g] = sgp->mask[g][min(mp, p.P - 1)];
    } else {
        mword = mask[min(mp, p.P - 1)];
    }
    int rword = 0;
    if (ADD) rword = rp.mask[min(mp, p.P - 1)];
    // SEG: tensor, first step and channel count of reduction step s (uniform selects: an indexed
    // read of the argument block would move it to scratch memory)
    auto seg_of = [&](int st) { return SEG ? (st >= sgp->step0[1]) + (st >= sgp->step0[2]) + (st >= sgp->step0[3]) : 0; };
    auto seg_in = [&](int g) { return g == 0 ? sgp->in[0] : g == 1 ? sgp->in[1] : g == 2 ? sgp->in[2] : sgp->in[3]; };
    auto seg_c = [&](int g) { return g == 0 ? sgp->C[0] : g == 1 ? sgp->C[1] : g == 2 ? sgp->C[2] : sgp->C[3]; };
    auto seg_s0 = [&](int g) { return g == 0 ? sgp->step0[0] : g == 1 ? sgp->step0[1] : g == 2 ? sgp->step0[2] : sgp->step0[3]; };
    // SEG: the input fragment of step st for pixel tile j of this wavefront (clamped pixel; what an
    // inactive pixel returns is zeroed before it is used)
    auto seg_x = [&](int st, int j) {
        const int g = seg_of(st);
        const size_t pix = (size_t)min(pbase + (nw * NTW + j) * 16 + l16, p.P - 1);
        return *reinterpret_cast<const E8 *>(seg_in(g) + pix * seg_c(g) + ((st - seg_s0(g)) << 5) + kq * 8);
    };
    const int ct0 = (by * CBW + cw) * R;
    const E *wrow[R];  // fragment order: one contiguous KB per (channel tile, step)
#pragma unroll
    for (int r = 0; r < R; ++r)  // surplus channel tiles re-read the last one and are not stored
        wrow[r] = wp + (size_t)min(ct0 + r, p.co_tiles - 1) * ksteps * 512 + lane * 8;
    E8 a[S][R];
#pragma unroll
    for (int i = 0; i < S; ++i) {
        const int s = min(kw + i * KW, ksteps - 1);
#pragma unroll
        for (int r = 0; r < R; ++r) a[i][r] = *reinterpret_cast<const E8 *>(wrow[r] + (s << 9));
    }
    // EAGER: the input fragments of the first chunk are requested before the masks are known
    // (one memory round trip less in the dependency chain; what inactive pixels return is
    // never stored)
    const E *xrow[NTW];
    E8 x[S][NTW];
    if (EAGER) {
#pragma unroll
        for (int j = 0; j < NTW; ++j)
            xrow[j] = SEG ? nullptr : in + (size_t)min(pbase + (nw * NTW + j) * 16 + l16, p.P - 1) * p.Ci;
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int s = min(kw + i * KW, ksteps - 1);
            const int k = min((s << 5) + kq * 8, p.Ci - 8);
#pragma unroll
            for (int j = 0; j < NTW; ++j) x[i][j] = SEG ? seg_x(s, j) : *reinterpret_cast<const E8 *>(xrow[j] + k);
        }
    }
    // tiles this wavefront finishes: all of its own (KW == 1) or tiles kw, kw + KW, ... of
    // its group after the reduction
    E4 res[FT], bh[FT], qv[FT];
    if (OPEN && EAGER) {  // the activation's cached state of the lane's pixels, before the masks are known
#pragma unroll
        for (int m = 0; m < FT; ++m) {
            const int t = min(KW > 1 ? kw + m * KW : m, TILES - 1);
            const int r = t / NTW, j = t % NTW;
            const int co = min((ct0 + r) * 16 + kq * 4, p.Co - 4);
            const size_t off = (size_t)min(pbase + (nw * NTW + j) * 16 + l16, p.P - 1) * p.Co + co;
            res[m] = *reinterpret_cast<const E4 *>(rp.res + off);
            qv[m] = *reinterpret_cast<const E4 *>(rp.prev + off);
        }
    }
    uint64_t bseg[PW_MAX_SEGS] = {0, 0, 0, 0};
    if (SEG) {
#pragma unroll
        for (int g = 0; g < PW_MAX_SEGS; ++g) bseg[g] = g < sgp->n ? ballot(mine && sword[g] != 0) : 0;
    }
    const uint64_t bm = SEG ? (bseg[0] | bseg[1] | bseg[2] | bseg[3]) : ballot(mine && mword != 0);
    const uint64_t br = ADD ? ballot(mine && rword != 0) : 0;
    const uint64_t bo = bm | br;
    if (by == 0 && wave == 0 && mine) out_mask[mp] = int((bo >> lane) & 1);
    if (bo == 0) return;  // the same for every wavefront of the workgroup
    auto seg_bits = [&](int g) { return g == 0 ? bseg[0] : g == 1 ? bseg[1] : g == 2 ? bseg[2] : bseg[3]; };
    if (OPEN && EAGER) {  // requested above, arrived with the mask words: not to be moved down to the epilogue
#pragma unroll
        for (int m = 0; m < FT; ++m) {
            DC_PIN(res[m]);
            DC_PIN(qv[m]);
        }
    }

#pragma unroll
    for (int m = 0; m < FT; ++m) {
        const int t = KW > 1 ? kw + m * KW : m;
        const int r = t / NTW, j = t % NTW;
        const int co = min((ct0 + r) * 16 + kq * 4, p.Co - 4);
        bh[m] = zero4<E>();
        if (bias != nullptr) bh[m] = *reinterpret_cast<const E4 *>(bias + co);
        if (ADD) {
            const int bit = (nw * NTW + j) * 16 + l16;
            const bool on_r = t < TILES && ((br >> bit) & 1);
            res[m] = *reinterpret_cast<const E4 *>(rp.res + (size_t)(on_r ? pbase + bit : 0) * p.Co + co);
            if (ADDACT) {
                const bool on_o = t < TILES && ((bo >> bit) & 1);
                qv[m] = *reinterpret_cast<const E4 *>(rp.prev + (size_t)(on_o ? pbase + bit : 0) * p.Co + co);
            }
        }
        if (OPEN && !EAGER) {  // cached state of the layer's activation, for updated pixels
            const int bit = (nw * NTW + j) * 16 + l16;
            const bool on_c = t < TILES && ((bm >> bit) & 1);
            const size_t off = (size_t)(on_c ? pbase + bit : 0) * p.Co + co;
            res[m] = *reinterpret_cast<const E4 *>(rp.res + off);
            qv[m] = *reinterpret_cast<const E4 *>(rp.prev + off);
        }
    }

    float4_t acc[R][NTW];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < NTW; ++j) acc[r][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    bool nt_on[NTW];
    bool wave_on = false;
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
        const int bit = (nw * NTW + j) * 16;
        nt_on[j] = ((bm >> bit) & 0xffffu) != 0;
        wave_on |= nt_on[j];
        // inactive pixels all point at pixel 0, so their (discarded) loads share one cache line
        if (!EAGER && !SEG) xrow[j] = in + (size_t)(((bm >> (bit + l16)) & 1) ? pbase + bit + l16 : 0) * p.Ci;
    }

    if (wave_on) {
        for (int s0 = kw; s0 < ksteps; s0 += S * KW) {
            if (s0 != kw) {
#pragma unroll
                for (int i = 0; i < S; ++i) {
                    const int s = min(s0 + i * KW, ksteps - 1);
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        a[i][r] = *reinterpret_cast<const E8 *>(wrow[r] + (s << 9));
                }
            }
            if (!EAGER || s0 != kw) {
#pragma unroll
                for (int i = 0; i < S; ++i) {
                    const int s = min(s0 + i * KW, ksteps - 1);
                    const int k = min((s << 5) + kq * 8, p.Ci - 8);
#pragma unroll
                    for (int j = 0; j < NTW; ++j) x[i][j] = SEG ? seg_x(s, j) : *reinterpret_cast<const E8 *>(xrow[j] + k);
                }
            }
            // No zero-fill is needed: columns of inactive pixels are never stored, and where a
            // step reaches past Cin the packed filter holds zeros while the clamped address
            // re-reads finite values of the same pixel.
#pragma unroll
            for (int i = 0; i < S; ++i) {
                if (s0 + i * KW < ksteps) {  // wave-uniform
                    const uint64_t sb = SEG ? seg_bits(seg_of(s0 + i * KW)) : 0;  // the step's tensor: its mask
#pragma unroll
                    for (int j = 0; j < NTW; ++j)
                        if (nt_on[j]) {  // wave-uniform
                            const E8 xz = SEG ? keep8(x[i][j], (sb >> ((nw * NTW + j) * 16 + l16)) & 1) : x[i][j];
#pragma unroll
                            for (int r = 0; r < R; ++r)
                                acc[r][j] = Elem16<E>::mfma(a[i][r], xz, acc[r][j]);
                        }
                }
            }
        }
    }

    float4_t fin[FT];
    if (KW > 1) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NTW; ++j) s_red[(wave * TILES + r * NTW + j) * WAVE + lane] = acc[r][j];
        __syncthreads();
#pragma unroll
        for (int m = 0; m < FT; ++m) {
            const int t = min(kw + m * KW, TILES - 1);
            float4_t sum = s_red[((tw * KW) * TILES + t) * WAVE + lane];
#pragma unroll
            for (int q = 1; q < KW; ++q) sum += s_red[((tw * KW + q) * TILES + t) * WAVE + lane];
            fin[m] = sum;
        }
    } else {
#pragma unroll
        for (int m = 0; m < FT; ++m) fin[m] = acc[m / NTW][m % NTW];
    }

    const E wa = E(rp.wa), wb = E(rp.wb);
    const int act = ACTC >= 0 ? ACTC : rp.act;
#pragma unroll
    for (int m = 0; m < FT; ++m) {
        const int t = KW > 1 ? kw + m * KW : m;
        if (t >= TILES) continue;
        const int r = t / NTW, j = t % NTW;
        const int ct = ct0 + r, co = ct * 16 + kq * 4;  // Cout % 4 == 0: a lane's 4 channels are all in or all out
        if (OPEN) {
            // D and T of the tile go through a wavefront-private LDS tile and leave as pieces of
            // pixel rows, 16 bytes per lane (Cout % 8 == 0): lanes 0..31 store D, lanes 32..63 T,
            // two neighbouring lanes one pixel's 16 channels.
            if (ct >= p.co_tiles) continue;  // the same for the whole wavefront
            const float4_t v = fin[m] + float4_t{float(bh[m][0]), float(bh[m][1]), float(bh[m][2]), float(bh[m][3])};
            E4 d, tq;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                tq[i] = res[m][i] + E(v[i]);
                const E sm = tq[i] + qv[m][i];
                d[i] = act_apply<E>(sm, act) - act_apply<E>(qv[m][i], act);
            }
            E *st = s_open + wave * 512;
            *reinterpret_cast<E4 *>(st + l16 * 16 + kq * 4) = d;
            *reinterpret_cast<E4 *>(st + 256 + l16 * 16 + kq * 4) = tq;
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const int which = lane >> 5, pr = (lane & 31) >> 1, hf = lane & 1;
            const int pbit = (nw * NTW + j) * 16 + pr, ch = ct * 16 + hf * 8;
            const E8 piece = *reinterpret_cast<const E8 *>(st + which * 256 + pr * 16 + hf * 8);
            if (((bm >> pbit) & 1) && ch < p.Co)
                *reinterpret_cast<E8 *>((which ? rp.tmp : out) + (size_t)(pbase + pbit) * p.Co + ch) = piece;
            if (FT > 1) {  // the tile is written again for the wavefront's next tile
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
            continue;
        }
        if (ct >= p.co_tiles || co >= p.Co) continue;
        const int bit = (nw * NTW + j) * 16 + l16;
        const bool on = (bm >> bit) & 1, on_r = (br >> bit) & 1;
        if (!(on || on_r)) continue;
        const float4_t v = fin[m] + float4_t{float(bh[m][0]), float(bh[m][1]), float(bh[m][2]), float(bh[m][3])};
        E4 o = E4{E(v[0]), E(v[1]), E(v[2]), E(v[3])};
        if (ADD) {  // add_kernel's sequence: s = a * wa; s = fma(b, wb, s); n = s + prev; ...
            E4 qn;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                E sum = on_r ? E(res[m][i] * wa) : E(0);
                if (on) sum = fma_t(o[i], wb, sum);
                if (ADDACT) {
                    qn[i] = sum + qv[m][i];
                    sum = act_apply<E>(qn[i], act) - act_apply<E>(qv[m][i], act);
                }
                o[i] = sum;
            }
            if (ADDACT) *reinterpret_cast<E4 *>(rp.prev + (size_t)(pbase + bit) * p.Co + co) = qn;
        }
        *reinterpret_cast<E4 *>(out + (size_t)(pbase + bit) * p.Co + co) = o;
    }
}

template <typename E, int KW, int CBW, int NBW, int R, int NTW, int S, int MODE, bool EAGER, int ACTC = -1>
__global__ void __launch_bounds__(KW * CBW * NBW * WAVE)
pw_mfma_kernel(PwP p, const E *__restrict__ in, const E *__restrict__ wp,
               const E *__restrict__ bias, E *__restrict__ out,
               const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, ResP<E> rp, PwSegs<E> sg) {
    __shared__ float4_t s_red[KW > 1 ? KW * CBW * NBW * R * NTW * WAVE : 1];
    // MODE 3: per wavefront one 16 x 16 tile each of D and T on their way into pixel rows
    __shared__ __align__(16) E s_open[MODE == 3 ? KW * CBW * NBW * 512 : 8];
    int bx = blockIdx.x, by = blockIdx.y;
    if (p.xcd) {
        const int slot = blockIdx.x >> 3;
        by = (blockIdx.x & 7) + 8 * (slot / p.nx);
        bx = slot % p.nx;
        if (by >= p.ny) return;  // padding of the channel groups to a multiple of 8
    }
    pw_mfma_body<E, KW, CBW, NBW, R, NTW, S, MODE, EAGER, ACTC>(p, in, wp, bias, out, mask, out_mask, rp, bx, by, s_red,
                                                                 s_open, &sg);
}

// Several independent small pointwise layers in ONE launch (the 1x1 convolutions of a
// multi-resolution exchange): a workgroup looks up the layer its number falls into and runs the
// one-tile, one-wavefront arrangement of pw_mfma_kernel on it unchanged, so the results are those
// of the separate launches bit for bit.  Plain convolutions whose own launch would use that
// arrangement only.
template <typename E>
struct PwItem {
    PwP p;
    const E *in, *wp, *bias;
    E *out;
    const int32_t *mask;
    int32_t *out_mask;
    int steps;  // fragment loads in flight together: 1, 2 or 4 reduction steps
    int nx;     // pixel tiles
    int first;  // number of this layer's first workgroup
};

template <typename E>
struct PwGroup {
    int n;
    PwItem<E> it[CONV_GROUP_MAX];
};

template <typename E>
__global__ void __launch_bounds__(WAVE)
pw_group_kernel(PwGroup<E> g) {
    int idx = 0;
#pragma unroll
    for (int i = 1; i < CONV_GROUP_MAX; ++i)
        if (i < g.n && (int)blockIdx.x >= g.it[i].first) idx = i;
    const PwItem<E> &it = g.it[idx];
    const int local = blockIdx.x - it.first;
    const int bx = local % it.nx, by = local / it.nx;
    const ResP<E> none{nullptr, nullptr, 1.f, 1.f, nullptr, 0};
    if (it.steps == 1)
        pw_mfma_body<E, 1, 1, 1, 1, 1, 1, 0, true>(it.p, it.in, it.wp, it.bias, it.out, it.mask, it.out_mask, none, bx, by, nullptr);
    else if (it.steps == 2)
        pw_mfma_body<E, 1, 1, 1, 1, 1, 2, 0, true>(it.p, it.in, it.wp, it.bias, it.out, it.mask, it.out_mask, none, bx, by, nullptr);
    else
        pw_mfma_body<E, 1, 1, 1, 1, 1, 4, 0, true>(it.p, it.in, it.wp, it.bias, it.out, it.mask, it.out_mask, none, bx, by, nullptr);
}

// --------------------------------------------------------------- fused conv + act/trunc
// Workgroup = NW wavefronts x 16 pixels x all output channels; wavefront w owns channel tiles
// w, w + NW, ... (at most CTW of them).  KS bounds the reduction steps: the input fragments of
// the 16 pixels stay in registers for the whole kernel and every loop is fully unrolled without
// branches (surplus steps multiply zero fragments, surplus tiles are computed and dropped), so
// the filter stream of a wavefront is one uninterrupted run of loads.  Requires Cout % 4 == 0.
// Pass 1 of the epilogue: conv output v (rounded to fp16), T = trunc + v, S = T + prev,
// D = act(S) - act(prev), one rounding each; collects the keep statistics of this lane.
template <typename E, int CTW, int ACT>
__device__ __forceinline__ void pw_epilogue_stats(const float4_t (&acc)[CTW], const typename Elem16<E>::v4 (&q)[CTW],
                                                  const typename Elem16<E>::v4 (&tr)[CTW], typename Elem16<E>::v4 (&v)[CTW],
                                                  const typename Elem16<E>::v4 (&bh)[CTW], bool on, int wave,
                                                  int NW, int kq, const PwP &p, E thr, bool norm,
                                                  bool &hit, float &sq) {
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        if (ct >= p.co_tiles) break;  // wave-uniform: surplus tiles of the last wavefronts
        const int co = ct * 16 + kq * 4;
        const bool live = co < p.Co;
        const float4_t r = acc[j] + float4_t{float(bh[j][0]), float(bh[j][1]), float(bh[j][2]), float(bh[j][3])};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[j][i] = E(r[i]);
            const E t = tr[j][i] + v[j][i];
            const E s = t + q[j][i];
            const E d = act_apply<E>(s, ACT) - act_apply<E>(q[j][i], ACT);
            if (live && on) {
                hit |= tabs(d) > thr;
                if (norm) sq += float(d) * float(d);  // uniform: only the norm modes need it
            }
        }
    }
}

// Pass 2: recompute T, S, D (a handful of ALU operations, cheaper than keeping them in
// registers across the workgroup barrier) and write the kept / dropped state.
template <typename E, int CTW, int ACT>
__device__ __forceinline__ void pw_epilogue_store(const typename Elem16<E>::v4 (&q)[CTW], const typename Elem16<E>::v4 (&tr)[CTW],
                                                  const typename Elem16<E>::v4 (&v)[CTW], bool keep, int wave, int NW,
                                                  int kq, int px, const PwP &p,
                                                  E *__restrict__ out, E *__restrict__ prev,
                                                  E *__restrict__ trunc) {
    typedef typename Elem16<E>::v4 E4;
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        if (ct >= p.co_tiles) break;  // wave-uniform
        const int co = ct * 16 + kq * 4;
        if (co >= p.Co) continue;
        const size_t off = (size_t)px * p.Co + co;
        E4 t, s, d;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            t[i] = tr[j][i] + v[j][i];
            s[i] = t[i] + q[j][i];
            d[i] = act_apply<E>(s[i], ACT) - act_apply<E>(q[j][i], ACT);
        }
        if (keep) {
            *reinterpret_cast<E4 *>(prev + off) = s;
            *reinterpret_cast<E4 *>(out + off) = d;
            if (bits_set8(tr[j])) *reinterpret_cast<E4 *>(trunc + off) = zero4<E>();  // else zero already
        } else {
            *reinterpret_cast<E4 *>(trunc + off) = t;
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
// w, w + NW, ... (at most CTW of them).  Everything whose address depends on coordinates only
// -- mask words, the first two reduction steps of filter and input fragments, the cached state
// and the bias of this lane's (pixel, 4 channel) cells -- is requested at once, so a layer with
// a reduction of up to 64 input channels is one memory round trip, the MFMAs, one barrier and
// the stores.  Longer reductions stream two steps per round trip in ascending order (the same
// summation order as the convolution-only kernel without reduction split).  What is loaded
// for inactive pixels is dropped.  Requires Cout % 4 == 0.
template <typename E, int NW, int CTW, int ACT>
__global__ void __launch_bounds__(NW * WAVE)
pw_act_mfma_kernel(PwP p, const E *__restrict__ in, const E *__restrict__ wp,
                   const E *__restrict__ bias, E *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                   E *__restrict__ prev, E *__restrict__ trunc, float thr_f, int mode) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int S = 2;
    __shared__ float s_stat[NW][16];
    const int wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int ksteps = p.ci_p >> 5;
    const int px = blockIdx.x * 16 + l16;
    const int pxc = min(px, p.P - 1);
    const int m = mask[pxc];
    // Every operand is requested before the mask word has arrived (the host uses this kernel
    // while the cached state of the whole map is a few MB: reading it for inactive pixels too
    // costs less than a second memory round trip).
    const int pl = pxc;
    const E *wrow[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j)
        wrow[j] = wp + (size_t)min(wave + j * NW, p.co_tiles - 1) * ksteps * 512 + lane * 8;
    const E *xrow = in + (size_t)pl * p.Ci;
    E8 a[S][CTW], x[S];
#pragma unroll
    for (int i = 0; i < S; ++i) {
        const int s = min(i, ksteps - 1);
        x[i] = *reinterpret_cast<const E8 *>(xrow + min((s << 5) + kq * 8, p.Ci - 8));
#pragma unroll
        for (int j = 0; j < CTW; ++j) a[i][j] = *reinterpret_cast<const E8 *>(wrow[j] + (s << 9));
    }
    E4 q[CTW], tr[CTW], bh[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int co = min(min(wave + j * NW, p.co_tiles - 1) * 16 + kq * 4, p.Co - 4);
        const size_t off = (size_t)pl * p.Co + co;
        q[j] = *reinterpret_cast<const E4 *>(prev + off);
        tr[j] = *reinterpret_cast<const E4 *>(trunc + off);
        bh[j] = zero4<E>();
        if (bias != nullptr) bh[j] = *reinterpret_cast<const E4 *>(bias + co);
    }
    // all of the above is in flight before anything is waited for
#pragma unroll
    for (int i = 0; i < S; ++i) {
        DC_PIN(x[i]);
#pragma unroll
        for (int j = 0; j < CTW; ++j) DC_PIN(a[i][j]);
    }
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        DC_PIN(q[j]);
        DC_PIN(tr[j]);
        DC_PIN(bh[j]);
    }
    const bool on = px < p.P && m != 0;
    if (ballot(on) == 0) {  // same 16 pixels in every wavefront: the whole workgroup leaves
        if (wave == 0 && kq == 0 && px < p.P) out_mask[px] = 0;
        return;
    }
    // no zero-fill: see pw_mfma_kernel (inactive columns are dropped, padded filter is zero)
    float4_t acc[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < ksteps; s0 += S) {
        if (s0 != 0) {
#pragma unroll
            for (int i = 0; i < S; ++i) {
                const int s = min(s0 + i, ksteps - 1);
                x[i] = *reinterpret_cast<const E8 *>(xrow + min((s << 5) + kq * 8, p.Ci - 8));
#pragma unroll
                for (int j = 0; j < CTW; ++j)
                    a[i][j] = *reinterpret_cast<const E8 *>(wrow[j] + (s << 9));
            }
#pragma unroll
            for (int i = 0; i < S; ++i) {
                DC_PIN(x[i]);
#pragma unroll
                for (int j = 0; j < CTW; ++j) DC_PIN(a[i][j]);
            }
        }
#pragma unroll
        for (int i = 0; i < S; ++i) {
            if (s0 + i < ksteps) {  // uniform
#pragma unroll
                for (int j = 0; j < CTW; ++j)
                    acc[j] = Elem16<E>::mfma(a[i][j], x[i], acc[j]);
            }
        }
    }
    const E thr = E(thr_f);
    E4 v[CTW];
    bool hit = false;
    float sq = 0.f;
    pw_epilogue_stats<E, CTW, ACT>(acc, q, tr, v, bh, on, wave, NW, kq, p, thr, mode != DC_TRUNC_MAX, hit, sq);
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
    pw_epilogue_store<E, CTW, ACT>(q, tr, v, keep, wave, NW, kq, px, p, out, prev, trunc);
}


// ------------------------------------------- fused conv + act/trunc, epilogue on pixel rows
// The fused form for layers too large for pw_act_mfma_kernel's 8-byte epilogue accesses (many
// streams in a batch: output maps beyond 4 MB) and too wide for pw_gather_kernel (more than 256
// output channels, filters beyond LDS): 16 consecutive pixels x all output channels per
// workgroup, NW wavefronts x CTW channel tiles each, filter fragments streamed by the wavefront
// that owns the tile (reduction steps ascending, one accumulator: the order of pw_mfma_kernel
// without reduction slices).  The rounded result is transposed through LDS into pixel rows and
// the activation / truncation (maximum norm) runs on rows in 16-byte pieces, the keep decision of
// a pixel meeting in an LDS flag.  The masks are read first and only updated pixels are touched:
// this kernel serves throughput, not the latency chain.  Requires Cout % 8 == 0.
template <typename E, int NW, int CTW, int ACT>
__global__ void __launch_bounds__(NW * WAVE)
pw_rows_act_kernel(PwP p, const E *__restrict__ in, const E *__restrict__ wp,
                   const E *__restrict__ bias, E *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                   E *__restrict__ prev, E *__restrict__ trunc, float thr_f) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NT = NW * WAVE, S = 2;
    constexpr int PIECES = (16 * CTW * NW * 2 + NT - 1) / NT;  // 16-byte pieces of the tile per thread
    extern __shared__ __align__(16) unsigned char s_rows[];   // [16][rowb]
    __shared__ int s_keep[16];
    const int tid = threadIdx.x, wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int ksteps = p.ci_p >> 5;
    const int rc = p.Co >> 3;                 // pieces per pixel row
    const int rowb = p.Co * 2 + 16;           // padded: rows start in different banks
    const int px = blockIdx.x * 16 + l16;
    const int pxc = min(px, p.P - 1);
    const bool on = px < p.P && mask[pxc] != 0;
    const uint64_t bon = ballot(on) & 0xffffull;  // the same 16 pixels in every wavefront
    if (bon == 0) {
        if (wave == 0 && kq == 0 && px < p.P) out_mask[px] = 0;
        return;
    }
    if (tid < 16) s_keep[tid] = 0;
    // rows of the cached state of updated pixels, requested before the contraction
    E8 qrow[PIECES], trow[PIECES];
    int64_t poff[PIECES];  // element offset of the piece in the map, -1: nothing to do
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int c = tid + i * NT;
        const int r = c / rc, cc = c - r * rc;
        const bool live = r < 16 && ((bon >> r) & 1);
        poff[i] = live ? ((int64_t)blockIdx.x * 16 + r) * p.Co + cc * 8 : -1;
        if (live) {
            qrow[i] = *reinterpret_cast<const E8 *>(prev + poff[i]);
            trow[i] = *reinterpret_cast<const E8 *>(trunc + poff[i]);
        }
    }
    const E *wrow[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j)
        wrow[j] = wp + (size_t)min(wave + j * NW, p.co_tiles - 1) * ksteps * 512 + lane * 8;
    // inactive pixels read an updated pixel's row (finite values; their columns are dropped)
    const int src = on ? pxc : blockIdx.x * 16 + (__ffsll((long long)bon) - 1);
    const E *xrow = in + (size_t)src * p.Ci;
    float4_t acc[CTW];
#pragma unroll
    for (int j = 0; j < CTW; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < ksteps; s0 += S) {
        E8 a[S][CTW], x[S];
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int sidx = min(s0 + i, ksteps - 1);
            x[i] = *reinterpret_cast<const E8 *>(xrow + min((sidx << 5) + kq * 8, p.Ci - 8));
#pragma unroll
            for (int j = 0; j < CTW; ++j) a[i][j] = *reinterpret_cast<const E8 *>(wrow[j] + (sidx << 9));
        }
#pragma unroll
        for (int i = 0; i < S; ++i) {
            if (s0 + i < ksteps) {  // uniform
#pragma unroll
                for (int j = 0; j < CTW; ++j) acc[j] = Elem16<E>::mfma(a[i][j], x[i], acc[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < CTW; ++j) {
        const int ct = wave + j * NW;
        if (ct >= p.co_tiles) break;  // uniform
        const int co = ct * 16 + kq * 4;
        if (co >= p.Co) continue;
        E4 bh = zero4<E>();
        if (bias != nullptr) bh = *reinterpret_cast<const E4 *>(bias + co);
        E4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = E(acc[j][i] + float(bh[i]));
        *reinterpret_cast<E4 *>(s_rows + l16 * rowb + co * 2) = v;
    }
    __syncthreads();
    const E thr = E(thr_f);
    E8 vrow[PIECES];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        if (poff[i] < 0) continue;
        const int c = tid + i * NT;
        const int r = c / rc, cc = c - r * rc;
        vrow[i] = *reinterpret_cast<const E8 *>(s_rows + r * rowb + cc * 16);
        bool hit = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const E t = trow[i][j] + vrow[i][j];
            const E sm = t + qrow[i][j];
            const E d = act_apply<E>(sm, ACT) - act_apply<E>(qrow[i][j], ACT);
            hit |= tabs(d) > thr;
        }
        if (hit) s_keep[r] = 1;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        if (poff[i] < 0) continue;
        const int c = tid + i * NT;
        const int r = c / rc, cc = c - r * rc;
        const bool keep = s_keep[r] != 0;
        if (cc == 0) out_mask[blockIdx.x * 16 + r] = keep ? 1 : 0;
        E8 tv, sv, dv, z;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            tv[j] = trow[i][j] + vrow[i][j];
            sv[j] = tv[j] + qrow[i][j];
            dv[j] = act_apply<E>(sv[j], ACT) - act_apply<E>(qrow[i][j], ACT);
            z[j] = E(0);
        }
        if (keep) {
            *reinterpret_cast<E8 *>(prev + poff[i]) = sv;
            *reinterpret_cast<E8 *>(out + poff[i]) = dv;
            if (bits_set16(trow[i])) *reinterpret_cast<E8 *>(trunc + poff[i]) = z;  // else zero already
        } else {
            *reinterpret_cast<E8 *>(trunc + poff[i]) = tv;
        }
    }
    // pixels of the tile without an update: mask word 0
    if (wave == 0 && kq == 0 && px < p.P && !on) out_mask[px] = 0;
}

// ----------------------------------------------------------- large maps: active-pixel gather
// On maps of tens of thousands of pixels and more (many video streams in a batch, large frames)
// the fixed runs of 64 pixels above spend most of their workgroups on runs without an update,
// and their 8-byte accesses per lane (the MFMA accumulator layout) reach a fraction of the
// memory bandwidth.  Here a workgroup of four wavefronts scans a span of the update mask,
// compacts the updated pixels into an LDS list, and every wavefront then takes 16 LISTED pixels
// at a time: their rows are gathered by index, contracted against the whole filter -- staged
// in LDS once per workgroup, at most 32 KB -- so a wavefront holds ALL output channels of its
// 16 pixels; the result is rounded, transposed through a wavefront-private LDS tile into pixel
// rows, and the rest runs on rows in 16-byte pieces: the plain store (MODE 0), or the
// activation / truncation of DCActivation with its keep decision per pixel (MODE 2, maximum-norm
// truncation: T = trunc + v, S = T + prev, D = act(S) - act(prev), one rounding each, the
// sequence of act_trunc_pixel).  Reduction steps run in ascending order in one accumulator, the
// order of pw_mfma_kernel without reduction slices, which is the arrangement the host would
// otherwise pick for the layers this kernel takes.  Requires Cout % 8 == 0.
constexpr int PWG_WAVES = 4;
constexpr int PWG_MAX_STEPS = 8;

template <typename E, int CT, int KSM, int MODE, int ACT>
__global__ void __launch_bounds__(PWG_WAVES * WAVE)
pw_gather_kernel(PwP p, const E *__restrict__ in, const E *__restrict__ wp, const E *__restrict__ bias,
                 E *__restrict__ out, const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                 E *__restrict__ prev, E *__restrict__ trunc, float thr_f, int span) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NT = PWG_WAVES * WAVE;
    constexpr int RC = CT * 2;  // 16-byte pieces of a pixel row held by CT channel tiles
    extern __shared__ __align__(16) unsigned char s_dyn[];
    __shared__ int s_n;
    __shared__ int s_keep[PWG_WAVES][16];
    const int ksteps = p.ci_p >> 5;
    const int wbytes = p.co_tiles * ksteps * 1024;
    const int rowb = CT * 32 + 16;  // bytes of a staged pixel row: padded, rows start in different banks
    E *s_w = reinterpret_cast<E *>(s_dyn);
    unsigned char *s_v = s_dyn + wbytes + wave_id() * 16 * rowb;
    int *s_list = reinterpret_cast<int *>(s_dyn + wbytes + PWG_WAVES * 16 * rowb);
    const int tid = threadIdx.x, wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int p0 = blockIdx.x * span;
    if (tid == 0) s_n = 0;
    // the filter, in fragment order as packed (contiguous), requested before the mask words
    for (int i = tid * 8; i < wbytes / 2; i += NT * 8)
        *reinterpret_cast<E8 *>(s_w + i) = *reinterpret_cast<const E8 *>(wp + i);
    __syncthreads();
    for (int q0 = 0; q0 < span; q0 += NT) {
        const int px = p0 + q0 + tid;
        const bool in_map = q0 + tid < span && px < p.P;
        const bool on = in_map && mask[min(px, p.P - 1)] != 0;
        if (in_map && (MODE == 0 || !on)) out_mask[px] = on ? 1 : 0;
        int cnt;
        const int rank = wave_rank(on, cnt);
        int base = 0;
        if (lane == 0 && cnt > 0) base = atomicAdd(&s_n, cnt);
        base = __shfl(base, 0, WAVE);
        if (on) s_list[base + rank] = px;
    }
    __syncthreads();
    const int n = s_n;
    const E thr = E(thr_f);
    for (int t0 = wave * 16; t0 < n; t0 += PWG_WAVES * 16) {
        const int nt = min(16, n - t0);            // listed pixels of this tile
        const int pix = s_list[t0 + min(l16, nt - 1)];  // surplus columns repeat a listed pixel and are dropped
        const E *xrow = in + (size_t)pix * p.Ci;
        E8 x[KSM];
#pragma unroll
        for (int ks = 0; ks < KSM; ++ks)
            if (ks < ksteps) x[ks] = *reinterpret_cast<const E8 *>(xrow + min((ks << 5) + kq * 8, p.Ci - 8));
        // rows of the cached state, in the 16-byte pieces the epilogue works on: piece c of the
        // tile is piece c % RC of pixel c / RC; requested now, used after the contraction
        constexpr int PIECES = (16 * RC + WAVE - 1) / WAVE;
        E8 qrow[MODE == 2 ? PIECES : 1], trow[MODE == 2 ? PIECES : 1];
        int ppix[PIECES], pcol[PIECES];
        bool pon[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int c = lane + i * WAVE;
            const int r = c / RC, cc = c - r * RC;
            pon[i] = r < nt && cc * 8 < p.Co;
            ppix[i] = s_list[t0 + min(r, nt - 1)];
            pcol[i] = min(cc * 8, p.Co - 8);
            if (MODE == 2) {
                const size_t off = (size_t)ppix[i] * p.Co + pcol[i];
                qrow[i] = *reinterpret_cast<const E8 *>(prev + off);
                trow[i] = *reinterpret_cast<const E8 *>(trunc + off);
            }
        }
        float4_t acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[ct] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSM; ++ks) {
            if (ks < ksteps) {  // uniform
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const int ctc = min(ct, p.co_tiles - 1);  // surplus tiles repeat the last one and are dropped
                    const E8 a = *reinterpret_cast<const E8 *>(s_w + (size_t)(ctc * ksteps + ks) * 512 + lane * 8);
                    acc[ct] = Elem16<E>::mfma(a, x[ks], acc[ct]);
                }
            }
        }
        // rounded result into the wavefront's LDS tile, pixel rows contiguous
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const int co = min(ct, p.co_tiles - 1) * 16 + kq * 4;
            E4 bh = zero4<E>();
            if (bias != nullptr) bh = *reinterpret_cast<const E4 *>(bias + min(co, p.Co - 4));
            E4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = E(acc[ct][i] + float(bh[i]));
            *reinterpret_cast<E4 *>(s_v + l16 * rowb + ct * 32 + kq * 8) = v;
        }
        if (MODE == 2 && lane < 16) s_keep[wave][lane] = 0;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        E8 vrow[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int r = min(lane + i * WAVE, 16 * RC - 1) / RC;
            vrow[i] = *reinterpret_cast<const E8 *>(s_v + r * rowb + pcol[i] * 2);
        }
        if (MODE == 0) {
#pragma unroll
            for (int i = 0; i < PIECES; ++i)
                if (pon[i]) *reinterpret_cast<E8 *>(out + (size_t)ppix[i] * p.Co + pcol[i]) = vrow[i];
        } else {
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                bool hit = false;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const E t = trow[i][j] + vrow[i][j];
                    const E sm = t + qrow[i][j];
                    const E d = act_apply<E>(sm, ACT) - act_apply<E>(qrow[i][j], ACT);
                    hit |= tabs(d) > thr;
                }
                if (pon[i] && hit) s_keep[wave][(lane + i * WAVE) / RC] = 1;
            }
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            // second pass: T, S, D again (a handful of operations, cheaper than holding them)
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int c = lane + i * WAVE;
                const int r = min(c, 16 * RC - 1) / RC;
                const bool keep = s_keep[wave][r] != 0;
                if (!pon[i]) continue;
                const size_t off = (size_t)ppix[i] * p.Co + pcol[i];
                if (c - r * RC == 0) out_mask[ppix[i]] = keep ? 1 : 0;
                E8 tv, sv, dv, z;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    tv[j] = trow[i][j] + vrow[i][j];
                    sv[j] = tv[j] + qrow[i][j];
                    dv[j] = act_apply<E>(sv[j], ACT) - act_apply<E>(qrow[i][j], ACT);
                    z[j] = E(0);
                }
                if (keep) {
                    *reinterpret_cast<E8 *>(prev + off) = sv;
                    *reinterpret_cast<E8 *>(out + off) = dv;
                    if (bits_set16(trow[i])) *reinterpret_cast<E8 *>(trunc + off) = z;  // else zero already
                } else {
                    *reinterpret_cast<E8 *>(trunc + off) = tv;
                }
            }
        }
        // the tile's LDS row buffer and keep flags are reused by the next tile of this wavefront
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace

bool pointwise_eligible(const dc_geometry &g, int dtype) {
    return (dtype == DC_F16 || dtype == DC_BF16) && g.groups == 1 && g.in_c % 8 == 0 && g.in_c >= 8 && g.out_c % 4 == 0 &&
           g.kernel_h == 1 &&
           g.kernel_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
           g.pad_left == 0 && g.pad_bottom == 0 && g.pad_right == 0;
}

// Wavefront arrangements of pw_mfma_kernel in use: id, KW, CBW, NBW, R, NTW, EAGER.
// Measured on MI355X over MobileNetV2's layers and 64x64x256 maps: small problems are bound by
// the dependent-latency chain and by how many compute units take part, so they run one
// 16x16 output tile per workgroup (ids 0, 2, 3: reduction over 1, 4 or 8 wavefronts) with eager
// input loads; large problems are bound by fragment traffic and reuse fragments in registers
// (ids 4, 5).
#define DC_PW_CONFIGS(X)                                                                     \
    X(0, 1, 1, 1, 1, 1, true) X(1, 1, 2, 2, 1, 1, true) X(2, 4, 1, 1, 1, 1, true)             \
    X(3, 8, 1, 1, 1, 1, true) X(4, 1, 2, 1, 2, 4, false) X(5, 4, 1, 1, 4, 4, false)

// The fused kernel takes reductions of at most PW_FUSED_MAX_STEPS steps in ascending order, and
// every arrangement chosen here for such a reduction has KW == 1, so a layer gets the same
// summation order with and without the fused epilogue.
constexpr int PW_FUSED_MAX_STEPS = 10;

int pick_config(const PwP &p, int ksteps) {
    const int64_t tiles = (int64_t)ceil_div(p.P, 16) * p.co_tiles;
    // 64 pixels x 64 channels per workgroup (every fragment used four times) from 2048 output
    // tiles on (from 1536 for reductions of 16 steps and more); for reductions short enough for
    // the fused kernel only where that kernel is not used (>= 4096 tiles), so that a layer keeps
    // one summation order
    if (p.co_tiles >= 4 && ((ksteps > PW_FUSED_MAX_STEPS && tiles >= 2048) || (ksteps >= 16 && tiles >= 1536) ||
                            (ksteps >= 4 && tiles >= 4096)))
        return 5;
    if (tiles >= 4096 && ksteps >= 2 && p.co_tiles >= 4) return 4;
    if (ksteps <= PW_FUSED_MAX_STEPS) return (ksteps <= 2 && p.P >= 4096 && p.co_tiles >= 2) ? 1 : 0;
    // long reductions: split over wavefronts while there are few tiles, one wavefront per tile
    // once the tiles alone fill the chip
    // (1280 -> 512 on 17 x 30, 1024 tiles: 13.1 us with one wavefront per tile, 11.3 us with eight
    // slices, 9.2 us with four)
    if (ksteps > 24) return tiles >= 2048 ? 0 : tiles >= 1024 ? 2 : 3;
    return tiles >= 1024 ? 0 : 2;
}

namespace {
int config_slices(int cfg) {
#define DC_PW_KW(ID, KW, CBW, NBW, R, NTW, EA) \
    if (cfg == ID) return KW;
    DC_PW_CONFIGS(DC_PW_KW)
#undef DC_PW_KW
    return 1;
}

// Shapes pw_gather_kernel takes: maps of 2^16 pixels and more, a filter of at most 32 KB with
// up to 8 reduction steps and 16 channel tiles, output rows in whole 16-byte pieces, LDS within
// 64 KB -- and only layers whose pw_mfma_kernel arrangement has no reduction slices, so that a
// layer keeps one summation order whichever kernel serves it (fused sums stay with pw_mfma_kernel).
int gather_tiles(const PwP &p, int ksteps) {
    if (p.P < (1 << 16) || p.Co % 8 != 0 || p.co_tiles > 16 || ksteps > PWG_MAX_STEPS) return 0;
    if (p.co_tiles * ksteps * 1024 > (32 << 10)) return 0;
    if (config_slices(pick_config(p, ksteps)) != 1) return 0;
    const int ct = p.co_tiles <= 4 ? p.co_tiles : p.co_tiles <= 6 ? 6 : p.co_tiles <= 8 ? 8 : p.co_tiles == 9 ? 9
                   : p.co_tiles <= 12 ? 12 : 16;
    return ct;
}
int gather_span(const PwP &p) { return p.P >= (1 << 19) ? 1024 : p.P >= (1 << 18) ? 512 : 256; }
size_t gather_lds(const PwP &p, int ksteps, int ct) {
    return (size_t)p.co_tiles * ksteps * 1024 + (size_t)PWG_WAVES * 16 * (ct * 32 + 16) + (size_t)gather_span(p) * 4;
}
}  // namespace

int pointwise_reduction_slices(int pixels, int in_c, int out_c) {
    PwP p;
    p.P = pixels;
    p.Ci = in_c;
    p.Co = out_c;
    p.ci_p = (in_c + 31) / 32 * 32;
    p.co_tiles = ceil_div(out_c, 16);
    p.xcd = p.nx = p.ny = 0;
    return config_slices(pick_config(p, p.ci_p / 32));
}

namespace {
template <typename E>
hipError_t launch_pointwise_t(const dc_geometry &g, const void *in, const void *packed,
                              const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                              const ActEpilogue *epi, bool *epilogue_done, const Residual *res,
                              hipStream_t s, const OpenAct *open = nullptr, const PwSegs<E> *segs = nullptr) {
    PwP p;
    p.P = g.batch * g.in_h * g.in_w;
    p.Ci = g.in_c;
    p.Co = g.out_c;
    p.ci_p = (g.in_c + 31) / 32 * 32;
    p.co_tiles = ceil_div(g.out_c, 16);
    p.xcd = 0;
    p.nx = p.ny = 0;
    const int ksteps = p.ci_p / 32;
    *epilogue_done = false;
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    // Large maps: active-pixel gather, with the activation / truncation as its epilogue where the
    // layer has one with maximum-norm truncation.
    const auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const int gct = (res == nullptr && open == nullptr && segs == nullptr && al16(in) && al16(out) && al16(packed)) ? gather_tiles(p, ksteps) : 0;
    if (gct > 0 && gather_lds(p, ksteps, gct) <= (64u << 10)) {
        const bool with_act = epi != nullptr && epi->mode == DC_TRUNC_MAX && epi->trunc != nullptr && al16(epi->prev) &&
                              al16(epi->trunc);
        const int span = gather_span(p);
        const size_t lds = gather_lds(p, ksteps, gct);
        dim3 grid(ceil_div(p.P, span));
        note_kernel("pw_gather_kernel");
#define DC_PWG_K(CTV, KSV)                                                                                        \
    do {                                                                                                         \
        if (with_act) {                                                                                          \
            DC_ACT_SWITCH(act, (pw_gather_kernel<E, CTV, KSV, 2, A><<<grid, PWG_WAVES * WAVE, lds, s>>>(          \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, (E *)epi->prev,  \
                (E *)epi->trunc, epi->thr, span)));                                                              \
        } else {                                                                                                 \
            pw_gather_kernel<E, CTV, KSV, 0, 0><<<grid, PWG_WAVES * WAVE, lds, s>>>(                             \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, nullptr,         \
                nullptr, 0.f, span);                                                                             \
        }                                                                                                        \
    } while (0)
#define DC_PWG(CTV)                                                                                              \
    do {                                                                                                         \
        if (ksteps <= 2) DC_PWG_K(CTV, 2);                                                                       \
        else DC_PWG_K(CTV, PWG_MAX_STEPS);                                                                       \
    } while (0)
        const int act = epi != nullptr && epi->act > 0 ? epi->act : 0;
        switch (gct) {
            case 1: DC_PWG(1); break;
            case 2: DC_PWG(2); break;
            case 3: DC_PWG(3); break;
            case 4: DC_PWG(4); break;
            case 6: DC_PWG(6); break;
            case 8: DC_PWG(8); break;
            case 9: DC_PWG(9); break;
            case 12: DC_PWG(12); break;
            default: DC_PWG(16); break;
        }
#undef DC_PWG_K
#undef DC_PWG
        *epilogue_done = with_act;
        return hipGetLastError();
    }
    // Fused epilogue: a workgroup owns all output channels of its 16 pixels (up to 16
    // wavefronts x 2 channel tiles), so it takes the keep / drop decision itself.  Only for maps
    // of at least 512 pixels: a smaller map gives too few workgroups, the whole filter then
    // streams through a handful of compute units and the two-launch form (channel tiles spread
    // over many workgroups) is faster.
    const bool fusable = res == nullptr && epi != nullptr && epi->mode >= 0 && g.out_c % 4 == 0 && al8(epi->prev) &&
                         al8(epi->trunc) && al8(out);
    // ... and not for large problems either: >= 4096 output tiles of 16x16 with a reduction of
    // several steps (there fragment traffic dominates, and the convolution-only kernel reuses
    // every fragment 4 times where a 16-pixel workgroup cannot), or an output map beyond 4 MB
    // (as with many streams in a batch: there the epilogue's 8-byte accesses per lane hold the
    // fused kernel at a quarter of the bandwidth the separate activation kernel reaches).
    const bool large = ((int64_t)ceil_div(p.P, 16) * p.co_tiles >= 4096 && ksteps >= 2) ||
                       (int64_t)p.P * p.Co * 2 > (4 << 20);
    // ... nor for filters beyond 32 KB, which every 16-pixel workgroup would stream in full
    const bool small_filter = (int64_t)p.ci_p * p.Co * 2 <= (32 << 10);
    // large layers with a filter of up to 128 KB: the fused form with its epilogue on pixel rows
    if (fusable && large && epi->mode == DC_TRUNC_MAX && p.Co % 8 == 0 && al16(epi->prev) && al16(epi->trunc) &&
        al16(out) && ksteps <= PW_FUSED_MAX_STEPS && p.P >= 4096 && p.co_tiles <= 64 &&
        (int64_t)p.ci_p * p.Co * 2 <= (128 << 10) && config_slices(pick_config(p, ksteps)) == 1) {
        dim3 grid(ceil_div(p.P, 16));
        const int act = epi->act < 0 ? 0 : epi->act;
        const size_t lds = (size_t)16 * (p.Co * 2 + 16);
        note_kernel("pw_rows_act_kernel");
#define DC_ROWS(NWV, CTWV)                                                                              \
    do {                                                                                              \
        DC_ACT_SWITCH(act, (pw_rows_act_kernel<E, NWV, CTWV, A><<<grid, NWV * WAVE, lds, s>>>(          \
                               p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask,  \
                               out_mask, (E *)epi->prev, (E *)epi->trunc, epi->thr)));                \
        *epilogue_done = true;                                                                        \
        return hipGetLastError();                                                                     \
    } while (0)
        if (p.co_tiles <= 4) DC_ROWS(4, 1);
        if (p.co_tiles <= 8) DC_ROWS(4, 2);
        if (p.co_tiles <= 12) DC_ROWS(4, 3);
        if (p.co_tiles <= 16) DC_ROWS(4, 4);
        if (p.co_tiles <= 24) DC_ROWS(8, 3);
        if (p.co_tiles <= 32) DC_ROWS(16, 2);
        if (p.co_tiles <= 40) DC_ROWS(8, 5);
        if (p.co_tiles <= 48) DC_ROWS(16, 3);
        DC_ROWS(16, 4);
#undef DC_ROWS
    }
    if (fusable && ksteps <= PW_FUSED_MAX_STEPS && p.P >= 512 && !large && small_filter) {
        dim3 grid(ceil_div(p.P, 16));
        const int act = epi->act < 0 ? 0 : epi->act;
        note_kernel("pw_act_mfma_kernel");
        // as many wavefronts as channel tiles, up to 16; then several tiles per wavefront
        const int nw = p.co_tiles <= 4 ? 4 : p.co_tiles <= 8 ? 8 : 16;
        const int ctw = ceil_div(p.co_tiles, nw);
#define DC_GO(NW, CTW)                                                                                \
    do {                                                                                              \
        DC_ACT_SWITCH(act, (pw_act_mfma_kernel<E, NW, CTW, A><<<grid, NW * WAVE, 0, s>>>(                \
                               p, (const E *)in, (const E *)packed, (const E *)bias,   \
                               (E *)out, mask, out_mask, (E *)epi->prev,                    \
                               (E *)epi->trunc, epi->thr, epi->mode)));                          \
        *epilogue_done = true;                                                                        \
        return hipGetLastError();                                                                     \
    } while (0)
        if (nw == 4) DC_GO(4, 1);
        if (nw == 8) DC_GO(8, 1);
        if (ctw == 1) DC_GO(16, 1);
        if (ctw == 2) DC_GO(16, 2);  // 32 KB of filter: at most 32 channel tiles
#undef DC_GO
    }
    PwSegs<E> sg{};
    if (segs != nullptr) sg = *segs;
    ResP<E> rp{nullptr, nullptr, 1.f, 1.f, nullptr, 0};
    if (res != nullptr) rp = ResP<E>{(const E *)res->values, res->mask, res->wa, res->wb, (E *)res->prev, res->act};
    if (open != nullptr)
        rp = ResP<E>{(const E *)open->trunc, nullptr, 1.f, 1.f, (E *)open->prev, open->act < 0 ? 0 : open->act, (E *)open->trunc};
    const int cfg = pick_config(p, ksteps);
    note_kernel("pw_mfma_kernel");
#define DC_PW_S(KW, CBW, NBW, R, NTW, EA, SS)                                                        \
    do {                                                                                             \
        p.nx = ceil_div(p.P, NBW * NTW * 16);                                                        \
        p.ny = ceil_div(p.co_tiles, CBW * R);                                                        \
        /* filter bytes dominate and the plain order would spread a channel group over XCDs */      \
        p.xcd = (p.nx % 8 != 0 && p.ny > 1 && (int64_t)p.ci_p * p.Co > (int64_t)p.P * p.Ci) ? 1 : 0; \
        dim3 grid(p.xcd ? p.nx * ((p.ny + 7) / 8 * 8) : p.nx, p.xcd ? 1 : p.ny);                     \
        if (segs != nullptr)                                                                         \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 4, EA><<<grid, KW * CBW * NBW * WAVE, 0, s>>>(     \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else if (open != nullptr && open->act == DC_ACT_RELU6)                                       \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 3, EA, DC_ACT_RELU6><<<grid, KW * CBW * NBW * WAVE, 0, s>>>( \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else if (open != nullptr)                                                                    \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 3, EA, DC_ACT_RELU><<<grid, KW * CBW * NBW * WAVE, 0, s>>>( \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else if (res != nullptr && res->act == DC_ACT_RELU)                                          \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 2, EA, DC_ACT_RELU><<<grid, KW * CBW * NBW * WAVE, 0, s>>>( \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else if (res != nullptr && res->act > 0)                                                     \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 2, EA><<<grid, KW * CBW * NBW * WAVE, 0, s>>>(     \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else if (res != nullptr)                                                                     \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 1, EA><<<grid, KW * CBW * NBW * WAVE, 0, s>>>(     \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
        else                                                                                         \
            pw_mfma_kernel<E, KW, CBW, NBW, R, NTW, SS, 0, EA><<<grid, KW * CBW * NBW * WAVE, 0, s>>>(     \
                p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, rp, sg); \
    } while (0)
#define DC_PW(ID, KW, CBW, NBW, R, NTW, EA)                                                          \
    case ID: {                                                                                       \
        const int need = ceil_div(ksteps, KW);                                                       \
        if (need <= 1) DC_PW_S(KW, CBW, NBW, R, NTW, EA, 1);                                         \
        else if (need <= 2) DC_PW_S(KW, CBW, NBW, R, NTW, EA, 2);                                    \
        else DC_PW_S(KW, CBW, NBW, R, NTW, EA, 4);                                                   \
        break;                                                                                       \
    }
    switch (cfg) {
        DC_PW_CONFIGS(DC_PW)
        default: return hipErrorInvalidValue;
    }
#undef DC_PW
#undef DC_PW_S
    return hipGetLastError();
}
}  // namespace

hipError_t launch_pointwise(const dc_geometry &g, const void *in, const void *packed,
                            const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                            const ActEpilogue *epi, bool *epilogue_done, const Residual *res,
                            int dtype, hipStream_t s) {
    if (dtype == DC_BF16)
        return launch_pointwise_t<bf16_t>(g, in, packed, bias, out, mask, out_mask, epi, epilogue_done, res, s);
    return launch_pointwise_t<half_t>(g, in, packed, bias, out, mask, out_mask, epi, epilogue_done, res, s);
}

// The pointwise convolution of a concatenation of n (2..4) delta tensors that is never formed
// (MODE 4 of pw_mfma_kernel): `g` describes the convolution of the concatenated tensor, whose
// arrangement -- and hence summation order -- the launch takes.
bool pointwise_concat_eligible(const dc_geometry &g, const int32_t *channels, int n, int dtype) {
    if (!pointwise_eligible(g, dtype) || n < 2 || n > PW_MAX_SEGS) return false;
    int total = 0;
    for (int i = 0; i < n; ++i) {
        if (channels[i] <= 0 || channels[i] % 32 != 0) return false;
        total += channels[i];
    }
    return total == g.in_c;
}

namespace {
template <typename E>
hipError_t pointwise_concat_t(const dc_geometry &g, const void *const *inputs, const int32_t *const *masks,
                              const int32_t *channels, int n, const void *packed, void *out, int32_t *out_mask,
                              hipStream_t s) {
    PwSegs<E> sg;
    int step = 0;
    for (int i = 0; i < PW_MAX_SEGS; ++i) {
        const int k = i < n ? i : 0;
        sg.in[i] = (const E *)inputs[k];
        sg.mask[i] = masks[k];
        sg.C[i] = channels[k];
        sg.step0[i] = i < n ? step : (1 << 30);  // never reached
        if (i < n) step += channels[i] / 32;
    }
    sg.n = n;
    bool unused = false;
    return launch_pointwise_t<E>(g, inputs[0], packed, nullptr, out, masks[0], out_mask, nullptr, &unused, nullptr, s,
                                 nullptr, &sg);
}
}  // namespace

hipError_t launch_pointwise_concat(const dc_geometry &g, const void *const *inputs, const int32_t *const *masks,
                                   const int32_t *channels, int n, const void *packed, void *out, int32_t *out_mask,
                                   int dtype, hipStream_t s) {
    if (dtype == DC_BF16) return pointwise_concat_t<bf16_t>(g, inputs, masks, channels, n, packed, out, out_mask, s);
    return pointwise_concat_t<half_t>(g, inputs, masks, channels, n, packed, out, out_mask, s);
}

// A plain pointwise convolution whose own launch is one wavefront per 16 x 16 output tile:
// what pw_group_kernel runs.
bool pointwise_group_item_eligible(const ConvGroupItem &c, int dtype) {
    if (c.packed == nullptr || c.res != nullptr || c.epi != nullptr || !pointwise_eligible(c.g, dtype)) return false;
    PwP p;
    p.P = c.g.batch * c.g.in_h * c.g.in_w;
    p.Ci = c.g.in_c;
    p.Co = c.g.out_c;
    p.ci_p = (c.g.in_c + 31) / 32 * 32;
    p.co_tiles = ceil_div(c.g.out_c, 16);
    p.xcd = p.nx = p.ny = 0;
    const int ksteps = p.ci_p / 32;
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    return p.P < (1 << 16) && pick_config(p, ksteps) == 0 && al8(c.out) && al8(c.bias);
}

namespace {
template <typename E>
hipError_t launch_pointwise_group_t(const ConvGroupItem *items, int n, hipStream_t s) {
    PwGroup<E> pg;
    pg.n = n;
    int blocks = 0;
    for (int i = 0; i < n; ++i) {
        const ConvGroupItem &c = items[i];
        PwItem<E> &it = pg.it[i];
        it.p.P = c.g.batch * c.g.in_h * c.g.in_w;
        it.p.Ci = c.g.in_c;
        it.p.Co = c.g.out_c;
        it.p.ci_p = (c.g.in_c + 31) / 32 * 32;
        it.p.co_tiles = ceil_div(c.g.out_c, 16);
        it.p.xcd = 0;
        it.p.nx = it.nx = ceil_div(it.p.P, 16);
        it.p.ny = it.p.co_tiles;
        it.in = (const E *)c.in; it.wp = (const E *)c.packed; it.bias = (const E *)c.bias;
        it.out = (E *)c.out; it.mask = c.mask; it.out_mask = c.out_mask;
        const int ksteps = it.p.ci_p / 32;
        it.steps = ksteps <= 1 ? 1 : ksteps <= 2 ? 2 : 4;
        it.first = blocks;
        blocks += it.nx * it.p.co_tiles;
    }
    for (int i = n; i < CONV_GROUP_MAX; ++i) pg.it[i] = pg.it[0];
    note_kernel("pw_group_kernel");
    pw_group_kernel<E><<<dim3((unsigned)blocks), WAVE, 0, s>>>(pg);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_pointwise_group(const ConvGroupItem *items, int n, int dtype, hipStream_t s) {
    if (dtype == DC_BF16) return launch_pointwise_group_t<bf16_t>(items, n, s);
    return launch_pointwise_group_t<half_t>(items, n, s);
}

// ReLU and ReLU6 (what the layers in front of depthwise convolutions use) are instantiated; output
// channels in multiples of 8: D and T leave as 16-byte pieces of pixel rows.
bool pointwise_open_eligible(const dc_geometry &g, int dtype, int activation) {
    return pointwise_eligible(g, dtype) && g.out_c % 8 == 0 && (activation == DC_ACT_RELU || activation == DC_ACT_RELU6);
}

// The pointwise convolution of a layer whose activation / truncation is left open (MODE 3 of
// pw_mfma_kernel): out = D, truncated = T on updated pixels, out_mask = the update mask.
hipError_t launch_pointwise_open(const dc_geometry &g, const void *in, const void *packed, void *out,
                                 const int32_t *mask, int32_t *out_mask, const OpenAct &open, int dtype,
                                 hipStream_t s) {
    bool unused = false;
    if (dtype == DC_BF16)
        return launch_pointwise_t<bf16_t>(g, in, packed, nullptr, out, mask, out_mask, nullptr, &unused, nullptr, s, &open);
    return launch_pointwise_t<half_t>(g, in, packed, nullptr, out, mask, out_mask, nullptr, &unused, nullptr, s, &open);
}

}  // namespace dc
