// Two consecutive pointwise (1x1, stride 1) delta convolutions of an inverted-residual network in
// ONE launch: the projection that ends a block (no activation; optionally followed by the
// block's residual sum, a DCAdd without activation) and the expansion that starts the next block,
// whose activation / truncation is left OPEN as in pw_mfma_kernel's MODE 3 (D and T are stored,
// the keep decision and the state commit belong to the depthwise kernel behind it,
// conv_dw_kernel<FIN>).
//
// On the 14x14 maps of such a network each of the two layers is a launch of two to three memory
// round trips around a handful of MFMAs; what this kernel saves is the second launch and the
// trip of the block output through memory.  The projection needs every hidden channel of a pixel
// and the expansion every channel of the block output, so a workgroup owns 16 pixels through both
// layers; the expansion's channel tiles are split over gridDim.y workgroups, each of which
// repeats the (small) projection of its pixels -- only workgroup y == 0 stores it.  A workgroup
// therefore streams the whole projection filter: the form exists for filters of a few tens of KB.
//
// Arithmetic and summation order are those of the stand-alone kernels for the same layers
// (pw_mfma_kernel with four interleaved reduction slices for the projection, slice kw taking
// steps kw, kw + 4, ..., partial sums added in ascending slice order -- or, for reductions of up
// to ten steps, one ascending reduction; one ascending reduction for the expansion; one rounding
// to the tensor type after each layer; the sum as in add_kernel), so every output, mask and
// state is bit-identical to the two separate calls.
#include "epilogue.hpp"

namespace dc {
namespace {

constexpr int PAIR_NW = 8;   // wavefronts per workgroup

struct PairP {
    int P;                  // pixels
    int Ch, ksteps1;        // projection input channels, reduction steps of 32
    int Cm, cm_tiles;       // block output channels (projection out = expansion in), tiles of 16
    int ksteps2;            // Cm / 32
    int Ce, ce_tiles;       // expansion output channels, tiles of 16
    float wa, wb;           // weights of the residual and of the convolution in the sum
};

template <typename E>
struct PairPtr {
    const E *in;            // hidden delta [P][Ch]
    const int32_t *mask;
    const E *w1;            // projection filter, fragment order
    const E *res;           // residual delta [P][Cm] (ADD)
    const int32_t *rmask;
    E *out1;                // block output delta [P][Cm]
    int32_t *out_mask1;
    const E *w2;            // expansion filter, fragment order
    E *prev2;               // expansion's accumulated values (read)
    E *trunc2;              // expansion's truncated values (T written)
    E *out2;                // expansion's activated delta D
    int32_t *out_mask2;
};

// KW: reduction slices of the projection.  KW == 4: wavefront = (slice kw, one of 2 groups of R1
// channel tiles); KW == 1: wavefront t takes channel tile t on its own (R1 == 1, up to 8 tiles).
// S1: steps per reduction slice (upper bound); S2: reduction steps of the expansion (upper
// bound); CT2: expansion channel tiles per wavefront.
template <typename E, int KW, int R1, int S1, int S2, int CT2, bool ADD, int ACT>
__global__ void __launch_bounds__(PAIR_NW * WAVE)
pw_pair_kernel(PairP p, PairPtr<E> q) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NW = PAIR_NW;
    static_assert(KW == 4 || (KW == 1 && R1 == 1), "four slices over two tile groups, or one tile per wavefront");
    // partial sums of the reduction slices; afterwards the staging rows of the expansion's results
    constexpr int RED = KW > 1 ? KW * 2 * R1 * WAVE * 16 : 0;
    constexpr int ROW2 = NW * CT2 * 32 + 16;  // bytes per staged pixel row: this workgroup's channels of D (or T)
    constexpr int STAGE = 2 * 16 * ROW2;
    __shared__ __align__(16) unsigned char s_buf[RED > STAGE ? RED : STAGE];
    float4_t *s_red = reinterpret_cast<float4_t *>(s_buf);
    extern __shared__ __align__(16) unsigned char s_y[];  // [16][Cm * 2 + 16]: block output rows
    const int tid = threadIdx.x;
    const int wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int kw = KW > 1 ? wave % KW : 0, cg = KW > 1 ? wave / KW : wave;
    const int pbase = blockIdx.x * 16;
    const int rowb = p.Cm * 2 + 16;

    // ---- every request that does not depend on the masks, at once
    const int mp = pbase + lane;
    const bool mine = lane < 16 && mp < p.P;
    const int mword = q.mask[min(mp, p.P - 1)];
    int rword = 0;
    if (ADD) rword = q.rmask[min(mp, p.P - 1)];
    const int pix = min(pbase + l16, p.P - 1);
    // projection: filter fragments of the group's R1 tiles and the input fragments, slice kw
    E8 a1[S1][R1], x1[S1];
    const E *xrow = q.in + (size_t)pix * p.Ch;
#pragma unroll
    for (int i = 0; i < S1; ++i) {
        const int s = min(kw + i * KW, p.ksteps1 - 1);
        x1[i] = *reinterpret_cast<const E8 *>(xrow + min((s << 5) + kq * 8, p.Ch - 8));
#pragma unroll
        for (int r = 0; r < R1; ++r) {
            const int ct = min(cg * R1 + r, p.cm_tiles - 1);
            a1[i][r] = *reinterpret_cast<const E8 *>(q.w1 + ((size_t)ct * p.ksteps1 + s) * 512 + lane * 8);
        }
    }
    // expansion: filter fragments of this wavefront's tiles, cached state of the lane's elements
    int ct2[CT2];
    E8 a2[CT2][S2];
    E4 tr2[CT2], pv2[CT2];
#pragma unroll
    for (int j = 0; j < CT2; ++j) {
        ct2[j] = (blockIdx.y * NW + wave) * CT2 + j;
        const int ct = min(ct2[j], p.ce_tiles - 1);
#pragma unroll
        for (int s = 0; s < S2; ++s)
            a2[j][s] = *reinterpret_cast<const E8 *>(q.w2 + ((size_t)ct * p.ksteps2 + min(s, p.ksteps2 - 1)) * 512 + lane * 8);
    }
    // the residual's values for the tile this wavefront finishes (tile `wave` of the projection)
    E4 rv = zero4<E>();
    if (ADD && wave < p.cm_tiles) rv = *reinterpret_cast<const E4 *>(q.res + (size_t)pix * p.Cm + wave * 16 + kq * 4);

    const uint64_t bm = ballot(mine && mword != 0);
    const uint64_t br = ADD ? ballot(mine && rword != 0) : 0;
    const uint64_t bo = bm | br;
    if (blockIdx.y == 0 && wave == 0 && mine) {
        q.out_mask1[mp] = int((bo >> lane) & 1);
        q.out_mask2[mp] = int((bo >> lane) & 1);
    }
    if (bo == 0) return;  // the same for every wavefront of the workgroup
    // the expansion's cached state, for workgroups with an update: needed two barriers from here
#pragma unroll
    for (int j = 0; j < CT2; ++j) {
        const size_t off = (size_t)pix * p.Ce + min(min(ct2[j], p.ce_tiles - 1) * 16 + kq * 4, p.Ce - 4);
        tr2[j] = *reinterpret_cast<const E4 *>(q.trunc2 + off);
        pv2[j] = *reinterpret_cast<const E4 *>(q.prev2 + off);
    }
#pragma unroll
    for (int j = 0; j < CT2; ++j) {  // arrived with the mask words: not to be moved down to the epilogue
#pragma unroll
        for (int s = 0; s < S2; ++s) DC_PIN(a2[j][s]);
    }
    if (ADD) DC_PIN(rv);

    // ---- projection: partial sums of slice kw for the group's tiles
    float4_t acc1[R1];
#pragma unroll
    for (int r = 0; r < R1; ++r) acc1[r] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (bm != 0) {
#pragma unroll
        for (int i = 0; i < S1; ++i) {
            if (kw + i * KW < p.ksteps1) {  // wave-uniform
#pragma unroll
                for (int r = 0; r < R1; ++r) acc1[r] = Elem16<E>::mfma(a1[i][r], x1[i], acc1[r]);
            }
        }
    }
    if (KW > 1) {
#pragma unroll
        for (int r = 0; r < R1; ++r) s_red[((kw * 2 + cg) * R1 + r) * WAVE + lane] = acc1[r];
        __syncthreads();
    }
    const bool on = (bm >> l16) & 1, on_r = (br >> l16) & 1;
    if (wave < p.cm_tiles) {  // wavefront t finishes projection tile t
        float4_t sum = acc1[0];
        if (KW > 1) {
            const int g = wave / R1, r = wave % R1;
            sum = s_red[((0 * 2 + g) * R1 + r) * WAVE + lane];
#pragma unroll
            for (int k = 1; k < KW; ++k) sum += s_red[((k * 2 + g) * R1 + r) * WAVE + lane];
        }
        const float4_t v = sum + float4_t{0.f, 0.f, 0.f, 0.f};  // the stand-alone kernel's (absent) bias
        E4 o = E4{E(v[0]), E(v[1]), E(v[2]), E(v[3])};
        if (ADD) {  // add_kernel's sequence: s = a * wa; s = fma(b, wb, s)
            const E wa = E(p.wa), wb = E(p.wb);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                E sum2 = on_r ? E(rv[i] * wa) : E(0);
                if (on) sum2 = fma_t(o[i], wb, sum2);
                o[i] = sum2;
            }
        }
        const int co = wave * 16 + kq * 4;
        *reinterpret_cast<E4 *>(s_y + l16 * rowb + co * 2) = o;
    }
    __syncthreads();
    // the block output leaves as whole rows in 16-byte pieces (workgroup y == 0 only)
    if (blockIdx.y == 0) {
        const int per_row = p.Cm >> 3;
        for (int c = tid; c < 16 * per_row; c += NW * WAVE) {
            const int r = c / per_row, cc = c - r * per_row;
            if ((bo >> r) & 1)
                *reinterpret_cast<E8 *>(q.out1 + (size_t)(pbase + r) * p.Cm + cc * 8) =
                    *reinterpret_cast<const E8 *>(s_y + r * rowb + cc * 16);
        }
    }

    // ---- expansion on the block output (updated pixels: bo), activation left open.  Results are
    // staged in LDS as pixel rows (D, then T) and leave in 16-byte pieces, neighbouring lanes
    // writing neighbouring pieces of a row.
#pragma unroll
    for (int j = 0; j < CT2; ++j) {
        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < S2; ++s) {
            if (s < p.ksteps2) {
                const E8 x = *reinterpret_cast<const E8 *>(s_y + l16 * rowb + ((s << 5) + kq * 8) * 2);
                acc = Elem16<E>::mfma(a2[j][s], x, acc);
            }
        }
        const float4_t v = acc + float4_t{0.f, 0.f, 0.f, 0.f};
        E4 tq, d;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const E o = E(v[i]);
            tq[i] = tr2[j][i] + o;
            const E sm = tq[i] + pv2[j][i];
            d[i] = act_apply<E>(sm, ACT) - act_apply<E>(pv2[j][i], ACT);
        }
        const int lc = (wave * CT2 + j) * 16 + kq * 4;  // channel within the workgroup's share
        *reinterpret_cast<E4 *>(s_buf + l16 * ROW2 + lc * 2) = d;
        *reinterpret_cast<E4 *>(s_buf + (16 + l16) * ROW2 + lc * 2) = tq;
    }
    __syncthreads();
    {
        constexpr int PER_ROW = NW * CT2 * 2;  // 16-byte pieces per staged row
        const int c0 = blockIdx.y * NW * CT2 * 16;  // first channel of this workgroup
        for (int c = tid; c < 2 * 16 * PER_ROW; c += NW * WAVE) {
            const int which = c / (16 * PER_ROW), rr = c - which * 16 * PER_ROW;
            const int r = rr / PER_ROW, cc = rr - r * PER_ROW;
            const int ch = c0 + cc * 8;
            if (ch >= p.Ce || !((bo >> r) & 1)) continue;
            E *dst = which == 0 ? q.out2 : q.trunc2;
            *reinterpret_cast<E8 *>(dst + (size_t)(pbase + r) * p.Ce + ch) =
                *reinterpret_cast<const E8 *>(s_buf + (which * 16 + r) * ROW2 + cc * 16);
        }
    }
}

template <typename E>
hipError_t pair_t(const PairP &p, const PairPtr<E> &q, int kw, bool add, int act, hipStream_t s) {
    const int r1 = ceil_div(p.cm_tiles, 2);
    const int s1 = ceil_div(p.ksteps1, kw);
    const int ct2 = 1;
    dim3 grid(ceil_div(p.P, 16), ceil_div(p.ce_tiles, PAIR_NW * ct2));
    const size_t lds = (size_t)16 * (p.Cm * 2 + 16);
    note_kernel("pw_pair_kernel");
#define DC_PAIR4(KWV, R1V, S1V, S2V, ADDV, ACTV)                                                   \
    do {                                                                                           \
        pw_pair_kernel<E, KWV, R1V, S1V, S2V, 1, ADDV, ACTV><<<grid, PAIR_NW * WAVE, lds, s>>>(p, q); \
        return hipGetLastError();                                                                  \
    } while (0)
#define DC_PAIR3(KWV, R1V, S1V, S2V)                                                               \
    do {                                                                                           \
        if (add && act == DC_ACT_RELU6) DC_PAIR4(KWV, R1V, S1V, S2V, true, DC_ACT_RELU6);           \
        if (add) DC_PAIR4(KWV, R1V, S1V, S2V, true, DC_ACT_RELU);                                  \
        if (act == DC_ACT_RELU6) DC_PAIR4(KWV, R1V, S1V, S2V, false, DC_ACT_RELU6);                 \
        DC_PAIR4(KWV, R1V, S1V, S2V, false, DC_ACT_RELU);                                          \
    } while (0)
    (void)ct2;
    if (kw == 1) {
        if (s1 <= 6) DC_PAIR3(1, 1, 6, 3);
        if (s1 <= 10) DC_PAIR3(1, 1, 10, 3);
        return hipErrorInvalidValue;
    }
    if (r1 <= 2 && s1 <= 3 && p.ksteps2 <= 2) DC_PAIR3(4, 2, 3, 2);
    if (r1 <= 3 && s1 <= 3 && p.ksteps2 <= 3) DC_PAIR3(4, 3, 3, 3);
    if (r1 <= 3 && s1 <= 5 && p.ksteps2 <= 3) DC_PAIR3(4, 3, 5, 3);
#undef DC_PAIR3
#undef DC_PAIR4
    return hipErrorInvalidValue;
}

}  // namespace

// Shapes the pair kernel takes: both layers as pw_mfma_kernel would run them stand-alone with
// four reduction slices or none (projection) and none (expansion); block output channels in
// whole reduction steps of 32, at most 6 channel tiles; projection reductions of at most 20
// steps; a projection filter of at most 128 KB, which every workgroup streams in full.
bool pointwise_pair_eligible(const dc_geometry &gp, int expand_channels, int activation, int dtype) {
    if (!pointwise_eligible(gp, dtype) || expand_channels <= 0 || expand_channels % 8 != 0) return false;
    if (activation != DC_ACT_RELU && activation != DC_ACT_RELU6) return false;
    const int P = gp.batch * gp.out_h * gp.out_w;
    const int Cm = gp.out_c;
    if (Cm % 32 != 0 || Cm > 96) return false;
    const int ksteps1 = ceil_div(gp.in_c, 32);
    if (ksteps1 > 20 || (int64_t)gp.in_c * Cm * 2 > (128 << 10)) return false;
    const int kw = pointwise_reduction_slices(P, gp.in_c, Cm);
    if (kw != 4 && !(kw == 1 && ksteps1 <= 10)) return false;
    if (pointwise_reduction_slices(P, Cm, expand_channels) != 1) return false;
    return true;
}

hipError_t launch_pointwise_pair(const dc_geometry &gp, const void *in, const int32_t *mask,
                                 const void *project_packed, const Residual *res, void *out, int32_t *out_mask,
                                 const void *expand_packed, int expand_channels, const OpenAct &open,
                                 void *expand_out, int32_t *expand_out_mask, int dtype, hipStream_t s) {
    PairP p;
    p.P = gp.batch * gp.out_h * gp.out_w;
    p.Ch = gp.in_c;
    p.ksteps1 = ceil_div(gp.in_c, 32);
    p.Cm = gp.out_c;
    p.cm_tiles = ceil_div(p.Cm, 16);
    p.ksteps2 = p.Cm >> 5;
    p.Ce = expand_channels;
    p.ce_tiles = ceil_div(p.Ce, 16);
    p.wa = res != nullptr ? res->wa : 1.f;
    p.wb = res != nullptr ? res->wb : 1.f;
    const int act = open.act;
    const int kw = pointwise_reduction_slices(p.P, gp.in_c, p.Cm);
    if (dtype == DC_BF16) {
        PairPtr<bf16_t> q{(const bf16_t *)in, mask, (const bf16_t *)project_packed,
                          res != nullptr ? (const bf16_t *)res->values : nullptr, res != nullptr ? res->mask : nullptr,
                          (bf16_t *)out, out_mask, (const bf16_t *)expand_packed, (bf16_t *)open.prev,
                          (bf16_t *)open.trunc, (bf16_t *)expand_out, expand_out_mask};
        return pair_t<bf16_t>(p, q, kw, res != nullptr, act, s);
    }
    PairPtr<half_t> q{(const half_t *)in, mask, (const half_t *)project_packed,
                      res != nullptr ? (const half_t *)res->values : nullptr, res != nullptr ? res->mask : nullptr,
                      (half_t *)out, out_mask, (const half_t *)expand_packed, (half_t *)open.prev,
                      (half_t *)open.trunc, (half_t *)expand_out, expand_out_mask};
    return pair_t<half_t>(p, q, kw, res != nullptr, act, s);
}

}  // namespace dc
