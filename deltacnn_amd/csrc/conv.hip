// Delta convolution and delta transposed convolution.
//
// Every kernel works on an 8x8 tile of output pixels per workgroup:
//   1. one lane per output pixel ORs the input mask over the filter window (the dilated
//      output mask), writes it, and the active output pixels of the tile are compacted with
//      ballot + popcount rank; a tile without active pixels ends here;
//   2. only the compacted pixels are computed.  Inactive or out-of-bounds inputs contribute
//      zero by selection (what a speculative load returns for them is discarded).
//
// conv_direct_kernel  any dtype / kernel / stride / dilation / groups, VALU, fp32 accumulate
// conv_mfma_kernel    fp16, groups == 1, Cin % 8 == 0: implicit GEMM on
//                     v_mfma_f32_16x16x32_f16 with rows = output channels (packed filter
//                     [Cout][tap][Cin]) and columns = compacted pixels (NHWC rows), so both
//                     operands are 16-byte row loads and the accumulator tile stores 4
//                     consecutive channels per lane
#include <atomic>

#include "epilogue.hpp"
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
                            if (ip[j] >= 0) acc[j] = __builtin_fmaf(float(inb[(size_t)ip[j] * p.Ci + cin0 + cg]), w, acc[j]);
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

// ------------------------------------------------------------------------------- depthwise
// One group of G lanes per OUTPUT pixel (grid = pixels x G): the group ballots the input mask
// over the window into a tap bit set (the dilated output mask is "any bit set"), then walks
// only the active taps with 16-byte channel vectors.  With ACT >= 0 the activation/truncation
// of the layer runs on the accumulators as an epilogue, so the convolution output never makes
// a round trip through memory and one launch is saved per layer.
struct EpiP {
    void *prev;
    void *trunc;
    float thr;
    int mode;
};

// The activation / truncation of the layer that PRODUCED this kernel's input, left open by
// that layer (see pw_mfma_kernel MODE 3): `in` holds D = act(S) - act(prev) for every pixel the
// producer's convolution updated (mask = its update mask), and the layer's truncated values
// already hold T = truncated + v for those pixels.
struct OpenActP {
    void *prev;
    void *trunc;
    float thr;
};

// EAGER (3x3 only, small maps): the nine input rows, the filter and the cached state are
// requested before the mask words have arrived -- their addresses depend on coordinates only --
// so the whole kernel is one memory round trip; what is loaded for inactive pixels is dropped.
// FIN (EAGER, padding 1; 1: stride 1, 2: stride 2): the producing layer's activation / truncation
// is finished here, which saves that layer's activation launch.  A window pixel counts as updated
// only if the producer's keep decision holds for it -- any |D| above the producer's threshold over
// all channels, which this lane group sees since it reads the pixel's whole row anyway -- and the
// group commits the producer's cached state of the input pixels it OWNS: with stride 1 its centre
// pixel, with stride 2 the 2 x 2 block (2 oy + {0, 1}, 2 ox + {0, 1}), taps (1, 1) .. (2, 2) of its
// window -- every input pixel is owned by exactly one group.  Kept: prev += T, truncated = 0;
// dropped: truncated = T, which it holds already.  Neighbouring groups read D and the update mask
// only, never that state, so nothing races.
template <typename T, int ITERS, int ACT, bool K3, bool EAGER, int FIN = 0>
__global__ void __launch_bounds__(256)
conv_dw_kernel(ConvP p, const T *__restrict__ in, const T *__restrict__ filter,
               const T *__restrict__ bias, T *__restrict__ out, const int32_t *__restrict__ mask,
               int32_t *__restrict__ out_mask, EpiP epi, int lg, OpenActP fin = OpenActP{}) {
    static_assert(!FIN || (K3 && EAGER), "the open activation is finished by the eager 3x3 form only");
    constexpr int N = Vec16<T>::N;
    const int G = 1 << lg;
    const int C = p.Ci;
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int po = gid >> lg, gl = gid & (G - 1);
    const int P_out = p.B * p.Ho * p.Wo;
    const bool valid = po < P_out;
    const int pc = min(po, P_out - 1);  // surplus groups of the last workgroup shadow the last pixel
    const int b = pc / (p.Ho * p.Wo);
    const int r = pc - b * p.Ho * p.Wo;
    const int oy = r / p.Wo, ox = r - oy * p.Wo;
    const int K2 = K3 ? 9 : p.Kh * p.Kw;
    const int Kw = K3 ? 3 : p.Kw;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const int glo = lane_id() & ~(G - 1);
    const uint64_t gmask = G >= WAVE ? ~0ull : ((1ull << G) - 1ull);

    Vec<T, N> ex[K3 && EAGER ? 9 : 1][ITERS], ew[K3 && EAGER ? 9 : 1][ITERS], q[ITERS], tr[ITERS];
    if (K3 && EAGER) {
        const int cy = oy, cx = ox;
        const T *inb = in + (size_t)b * p.Hi * p.Wi * C;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int ky = t / 3, kx = t - ky * 3;
            const int iy = min(max(cy * p.sh - p.pt + ky * p.dh, 0), p.Hi - 1);
            const int ix = min(max(cx * p.sw - p.pl + kx * p.dw, 0), p.Wi - 1);
            const T *xr = inb + (size_t)(iy * p.Wi + ix) * C;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = min((it * G + gl) * N, C - N);
                ex[t][it] = vload<T, N>(xr + c);
                ew[t][it] = vload<T, N>(filter + (size_t)t * C + c);
            }
        }
        if (ACT >= 0) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = min((it * G + gl) * N, C - N);
                q[it] = vload<T, N>((const T *)epi.prev + (size_t)pc * C + c);
                tr[it] = vload<T, N>((const T *)epi.trunc + (size_t)pc * C + c);
            }
        }
    }
    // FIN: T and the accumulated value of the owned input pixels (padding 1: tap (1 + dy, 1 + dx) of
    // the window is input pixel (oy * stride + dy, ox * stride + dx)), requested with everything else
    constexpr int NOWN = FIN == 2 ? 4 : 1;
    Vec<T, N> ft[FIN ? NOWN : 1][FIN ? ITERS : 1], fq[FIN ? NOWN : 1][FIN ? ITERS : 1];
    size_t own[NOWN];
#pragma unroll
    for (int o = 0; o < NOWN; ++o)  // (past the map's edge: the edge pixel again; its tap is never set)
        own[o] = ((size_t)b * p.Hi + min(oy * (FIN == 2 ? 2 : 1) + (o >> 1), p.Hi - 1)) * p.Wi +
                 min(ox * (FIN == 2 ? 2 : 1) + (o & 1), p.Wi - 1);
    if (FIN) {
#pragma unroll
        for (int o = 0; o < NOWN; ++o)
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = min((it * G + gl) * N, C - N);
                ft[o][it] = vload<T, N>((const T *)fin.trunc + own[o] * C + c);
                fq[o][it] = vload<T, N>((const T *)fin.prev + own[o] * C + c);
            }
    }

    uint64_t taps = 0;
    const int GW = G > WAVE ? WAVE : G;  // a group wider than a wavefront: every wavefront scans
    for (int j = 0; j < K2; j += GW) {
        const int t = j + (gl & (GW - 1));
        bool m = false;
        if (valid && t < K2) {
            const int ky = t / Kw, kx = t - ky * Kw;
            const int iy = oy * p.sh - p.pt + ky * p.dh, ix = ox * p.sw - p.pl + kx * p.dw;
            if (iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi) m = mb[iy * p.Wi + ix] != 0;
        }
        taps |= ((ballot(m) >> glo) & gmask) << j;
    }
    if (FIN) {
        // (the centre pixel's state was requested with everything else and has arrived with the
        // mask words: keep the compiler from moving those requests down to the commit below)
#pragma unroll
        for (int o = 0; o < NOWN; ++o)
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                pin_vec(ft[o][it]);
                pin_vec(fq[o][it]);
            }
        // the producer's keep decision for the nine window pixels: this lane's share first (what
        // was loaded for a pixel without update is dropped), then the group's, straight-line
        const float fthr = float(T(fin.thr));
        uint32_t mine = 0;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            float big = 0.f;
#pragma unroll
            for (int it = 0; it < ITERS; ++it) big = fmaxf(big, vec_absmax(ex[t][it]));
            mine |= (big > fthr ? 1u : 0u) << t;
        }
        mine &= (uint32_t)taps;
        uint64_t kept = 0;
        if (G >= WAVE) {
#pragma unroll
            for (int t = 0; t < 9; ++t) kept |= (ballot((mine >> t) & 1u) != 0 ? 1ull : 0ull) << t;
        } else {
#pragma unroll
            for (int t = 0; t < 9; ++t) kept |= (((ballot((mine >> t) & 1u) >> glo) & gmask) != 0 ? 1ull : 0ull) << t;
        }
        if (G > WAVE) {  // one pixel per workgroup: the wavefronts hold different channels
            __shared__ uint32_t s_kept[4];
            if (lane_id() == 0) s_kept[wave_id()] = (uint32_t)kept;
            __syncthreads();
            kept = 0;
            for (int w = 0; w < (int)(blockDim.x / WAVE); ++w) kept |= s_kept[w];
        }
        // (a tap that was not updated is clear in `taps`, one that was not kept in `kept`)
        taps &= kept;
#pragma unroll
        for (int o = 0; o < NOWN; ++o) {
            const int tap = (1 + (o >> 1)) * 3 + 1 + (o & 1);  // 4; stride 2: 4, 5, 7, 8
            if (valid && ((taps >> tap) & 1ull)) {  // updated and kept
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int c = (it * G + gl) * N;
                    if (c < C) {
                        Vec<T, N> z, sum;
#pragma unroll
                        for (int j = 0; j < N; ++j) {
                            z.v[j] = T(0);
                            sum.v[j] = ft[o][it].v[j] + fq[o][it].v[j];
                        }
                        vstore<T, N>((T *)fin.prev + own[o] * C + c, sum);
                        vstore<T, N>((T *)fin.trunc + own[o] * C + c, z);
                    }
                }
            }
        }
    }
    const bool active = valid && taps != 0;
    if (valid && gl == 0) out_mask[po] = active ? 1 : 0;
    if (ballot(active) == 0) return;

    // cached state of the epilogue: requested now so that it arrives while the taps are summed
    if (ACT >= 0 && !(K3 && EAGER))
        load_state<T, ITERS>(q, tr, active, (size_t)po, gl, G, C, (const T *)epi.prev,
                             (const T *)epi.trunc);

    float acc[ITERS][N];
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int j = 0; j < N; ++j) acc[it][j] = 0.f;
    if (active) {
        const T *inb = in + (size_t)b * p.Hi * p.Wi * C;
        if (K3 && EAGER) {
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const bool on = (taps >> t) & 1ull;
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const Vec<T, N> xs = vkeep<T, N>(ex[t][it], on);
#pragma unroll
                    for (int j = 0; j < N; ++j)
                        acc[it][j] = __builtin_fmaf(float(xs.v[j]), float(ew[t][it].v[j]), acc[it][j]);
                }
            }
        } else if (K3 && ITERS <= 2) {
            // 3x3: every tap is loaded unconditionally from a clamped (always valid) address
            // and zeroed afterwards if the tap is inactive, so all loads are in flight
            // together: one memory round trip instead of one per tap
            Vec<T, N> x[9][ITERS], w[9][ITERS];
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const int ky = t / 3, kx = t - ky * 3;
                const int iy = min(max(oy * p.sh - p.pt + ky * p.dh, 0), p.Hi - 1);
                const int ix = min(max(ox * p.sw - p.pl + kx * p.dw, 0), p.Wi - 1);
                const T *xr = inb + (size_t)(iy * p.Wi + ix) * C;
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int c = min((it * G + gl) * N, C - N);
                    x[t][it] = vload<T, N>(xr + c);
                    w[t][it] = vload<T, N>(filter + (size_t)t * C + c);
                }
            }
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const bool on = (taps >> t) & 1ull;
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const Vec<T, N> xs = vkeep<T, N>(x[t][it], on);
#pragma unroll
                    for (int j = 0; j < N; ++j)
                        acc[it][j] = __builtin_fmaf(float(xs.v[j]), float(w[t][it].v[j]), acc[it][j]);
                }
            }
        } else {
            for (int t = 0; t < K2; ++t) {
                if (!((taps >> t) & 1ull)) continue;
                const int ky = t / p.Kw, kx = t - ky * p.Kw;
                const int iy = oy * p.sh - p.pt + ky * p.dh, ix = ox * p.sw - p.pl + kx * p.dw;
                const T *xr = inb + (size_t)(iy * p.Wi + ix) * C;
                const T *wr = filter + (size_t)t * C;
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int c = (it * G + gl) * N;
                    if (c < C) {
                        const Vec<T, N> x = vload<T, N>(xr + c);
                        const Vec<T, N> w = vload<T, N>(wr + c);
#pragma unroll
                        for (int j = 0; j < N; ++j)
                            acc[it][j] = __builtin_fmaf(float(x.v[j]), float(w.v[j]), acc[it][j]);
                    }
                }
            }
        }
    }
    Vec<T, N> dl[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int c = (it * G + gl) * N;
        if (active && c < C) {
            if (bias != nullptr) {
                const Vec<T, N> bv = vload<T, N>(bias + c);
#pragma unroll
                for (int j = 0; j < N; ++j) acc[it][j] += float(bv.v[j]);
            }
#pragma unroll
            for (int j = 0; j < N; ++j) dl[it].v[j] = T(acc[it][j]);
        }
    }
    if (ACT < 0) {
        if (active) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int c = (it * G + gl) * N;
                if (c < C) vstore<T, N>(out + (size_t)po * C + c, dl[it]);
            }
        }
    } else {
        act_trunc_pixel<T, ITERS, (ACT < 0 ? 0 : ACT)>(dl, q, tr, active, (size_t)po, gl, G, C, out,
                                                         (T *)epi.prev, (T *)epi.trunc, out_mask,
                                                         T(epi.thr), epi.mode);
    }
}

// Depthwise 3x3, stride 1, on maps of 4 MB and more (bandwidth regime): one group of lanes computes a strip
// of PX consecutive output pixels of a row.  The 3 x (PX + 2) input rows of the strip are
// loaded once (instead of 9 per pixel) and the filter stays in registers for the whole strip,
// which cuts load instructions and conversions per output pixel by more than half.  Per pixel
// the arithmetic (tap order, zero-select of inactive taps, bias, epilogue) is that of
// conv_dw_kernel, so the results are identical.
template <typename T, int ACT, bool LW>
__global__ void __launch_bounds__(256)
conv_dw_strip_kernel(ConvP p, const T *__restrict__ in, const T *__restrict__ filter,
                     const T *__restrict__ bias, T *__restrict__ out,
                     const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, EpiP epi,
                     int lg) {
    constexpr int N = Vec16<T>::N;
    constexpr int PX = 4, COLS = PX + 2, WORDS = 3 * COLS;
    const int G = 1 << lg;
    const int C = p.Ci;
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int sidx = gid >> lg, gl = gid & (G - 1);
    const int SW = (p.Wo + PX - 1) / PX;  // strips per row
    const int total = p.B * p.Ho * SW;
    const bool valid = sidx < total;
    const int sc = min(sidx, total - 1);  // surplus groups of the last workgroup shadow the last strip
    const int b = sc / (p.Ho * SW);
    const int r = sc - b * p.Ho * SW;
    const int oy = r / SW, ox0 = (r - oy * SW) * PX;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const int glo = lane_id() & ~(G - 1);
    const uint64_t gmask = G >= WAVE ? ~0ull : ((1ull << G) - 1ull);
    const int iy0 = oy - p.pt, ix0 = ox0 - p.pl;

    // LW: the filter goes through LDS once per workgroup, 36 registers less per lane (a third
    // wavefront per SIMD); costs a barrier, which small maps do not earn back
    __shared__ Vec<T, N> s_w[LW ? 9 : 1][WAVE];
    if (LW) {
        const int nv = C / N;
        for (int i = threadIdx.x; i < 9 * nv; i += 256) {
            const int t = i / nv, v = i - t * nv;
            s_w[t][v] = vload<T, N>(filter + (size_t)t * C + v * N);
        }
    }

    // activity of the 3 x COLS input pixels of the strip, one mask word per lane and pass
    uint32_t words = 0;
    for (int j = 0; j < WORDS; j += G) {
        const int w = j + gl;
        bool m = false;
        if (valid && w < WORDS) {
            const int wy = w / COLS, wx = w - wy * COLS;
            const int iy = iy0 + wy, ix = ix0 + wx;
            if (iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi) m = mb[iy * p.Wi + ix] != 0;
        }
        words |= (uint32_t)((ballot(m) >> glo) & gmask) << j;
    }
    uint32_t taps[PX];
    bool active[PX];
    bool any = false;
    const size_t po0 = ((size_t)b * p.Ho + oy) * p.Wo + ox0;
#pragma unroll
    for (int j = 0; j < PX; ++j) {
        taps[j] = ((words >> j) & 7u) | (((words >> (COLS + j)) & 7u) << 3) | (((words >> (2 * COLS + j)) & 7u) << 6);
        active[j] = valid && ox0 + j < p.Wo && taps[j] != 0;
        any |= active[j];
        if (valid && ox0 + j < p.Wo && gl == 0) out_mask[po0 + j] = active[j] ? 1 : 0;
    }
    if (LW) __syncthreads();
    if (ballot(any) == 0) return;

    const int c = min(gl * N, C - N);
    const bool lane_on = gl * N < C;
    Vec<T, N> q[PX][1], tr[PX][1];
    if (ACT >= 0) {
#pragma unroll
        for (int j = 0; j < PX; ++j)
            load_state<T, 1>(q[j], tr[j], active[j], po0 + j, gl, G, C, (const T *)epi.prev, (const T *)epi.trunc);
    }
    // all rows of the strip and the filter are requested together (clamped, always valid
    // addresses); inactive taps are zeroed by selection afterwards
    Vec<T, N> x[3][COLS];
    const T *inb = in + (size_t)b * p.Hi * p.Wi * C;
#pragma unroll
    for (int wy = 0; wy < 3; ++wy) {
        const int iy = min(max(iy0 + wy, 0), p.Hi - 1);
#pragma unroll
        for (int wx = 0; wx < COLS; ++wx) {
            const int ix = min(max(ix0 + wx, 0), p.Wi - 1);
            x[wy][wx] = vload<T, N>(inb + (size_t)(iy * p.Wi + ix) * C + c);
        }
    }
    Vec<T, N> w[LW ? 1 : 9];
    if (!LW) {
#pragma unroll
        for (int t = 0; t < 9; ++t) w[LW ? 0 : t] = vload<T, N>(filter + (size_t)t * C + c);
    }
    Vec<T, N> bv;
    if (bias != nullptr) bv = vload<T, N>(bias + c);

#pragma unroll
    for (int j = 0; j < PX; ++j) {
        float acc[N];
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] = 0.f;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const Vec<T, N> xs = vkeep<T, N>(x[t / 3][j + t % 3], (taps[j] >> t) & 1u);
            const Vec<T, N> wt = LW ? s_w[LW ? t : 0][c / N] : w[LW ? 0 : t];
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] = __builtin_fmaf(float(xs.v[e]), float(wt.v[e]), acc[e]);
        }
        Vec<T, N> dl[1];
        if (bias != nullptr) {
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] += float(bv.v[e]);
        }
#pragma unroll
        for (int e = 0; e < N; ++e) dl[0].v[e] = T(acc[e]);
        if (ACT < 0) {
            if (active[j] && lane_on) vstore<T, N>(out + (po0 + j) * C + c, dl[0]);
        } else {
            act_trunc_pixel<T, 1, (ACT < 0 ? 0 : ACT)>(dl, q[j], tr[j], active[j], po0 + j, gl, G, C, out,
                                                        (T *)epi.prev, (T *)epi.trunc, out_mask,
                                                        T(epi.thr), epi.mode);
        }
    }
}


// Depthwise 3x3 on maps of at least 2^18 outputs, any update density: a wavefront owns 64
// consecutive output pixels, one per lane while the nine mask words of the window are read and
// the output mask is written; the updated outputs are listed in LDS -- pixel, coordinates and the
// set of updated taps -- and served U at a time per lane group (one 16-byte vector per lane).
// A sparse map costs no idle lane groups, and the delta of a tap that was not updated is not
// fetched (its request goes to an updated tap's row, which is being read anyway).  The filter
// of the lane's channels is loaded once: into registers, or (LW) by the workgroup into LDS,
// which leaves room for more wavefronts per SIMD.  Per pixel the arithmetic is that of
// conv_dw_kernel.
template <typename T, int ACT, int U, bool LW>
__global__ void __launch_bounds__(256)
conv_dw_scan_kernel(ConvP p, const T *__restrict__ in, const T *__restrict__ filter,
                    const T *__restrict__ bias, T *__restrict__ out,
                    const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, EpiP epi,
                    int lg) {
    constexpr int N = Vec16<T>::N;
    __shared__ int s_pix[4][WAVE], s_yx[4][WAVE], s_img[4][WAVE], s_taps[4][WAVE];
    __shared__ Vec<T, N> s_w[LW ? 9 : 1][WAVE];
    const int Po = p.B * p.Ho * p.Wo, C = p.Ci;
    const int wave = wave_id(), lane = lane_id();
    const int po = (blockIdx.x * 4 + wave) * WAVE + lane;
    if (LW) {
        const int nv = C / N;
        for (int i = threadIdx.x; i < 9 * nv; i += 256) {
            const int t = i / nv, v = i - t * nv;
            s_w[t][v] = vload<T, N>(filter + (size_t)t * C + v * N);
        }
    }
    int taps = 0;  // bit t: tap t is inside the map and updated
    int yx, img;
    {
        const int pc = min(po, Po - 1);
        const int row = pc / p.Wo, ox = pc - row * p.Wo;
        const int b = row / p.Ho, oy = row - b * p.Ho;
        yx = (oy << 16) | ox;
        img = b * p.Hi * p.Wi;
        int mw[9];
        bool inside[9];
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int iy = oy * p.sh - p.pt + (t / 3) * p.dh, ix = ox * p.sw - p.pl + (t % 3) * p.dw;
            inside[t] = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
            mw[t] = mask[(size_t)img + min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1)];
        }
#pragma unroll
        for (int t = 0; t < 9; ++t) taps |= (inside[t] && mw[t] != 0) ? 1 << t : 0;
    }
    if (po >= Po) taps = 0;
    if (po < Po) out_mask[po] = taps != 0 ? 1 : 0;
    if (LW) __syncthreads();
    int n;
    const int rank = wave_rank(taps != 0, n);
    if (n == 0) return;
    if (taps != 0) {
        s_pix[wave][rank] = po;
        s_yx[wave][rank] = yx;
        s_img[wave][rank] = img;
        s_taps[wave][rank] = taps;
    }
    const int G = 1 << lg, gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    const bool mine = gl * N < C;
    const int c = min(gl * N, C - N);
    Vec<T, N> w[LW ? 1 : 9], bv;
    if (!LW) {
#pragma unroll
        for (int t = 0; t < 9; ++t) w[LW ? 0 : t] = vload<T, N>(filter + (size_t)t * C + c);
    }
    if (bias != nullptr) bv = vload<T, N>(bias + c);
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> x[U][9], q[U][1], tr[U][1];
        bool valid[U];
        int pix[U], tp[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp, e = min(idx, n - 1);
            valid[u] = idx < n && mine;
            pix[u] = s_pix[wave][e];
            tp[u] = s_taps[wave][e];
            const int oy = s_yx[wave][e] >> 16, ox = s_yx[wave][e] & 0xffff;
            const size_t base = (size_t)s_img[wave][e];
            const int first = __builtin_ctz(tp[u]);  // an updated tap: the list holds no other pixels
            size_t ip[9];
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const int iy = min(max(oy * p.sh - p.pt + (t / 3) * p.dh, 0), p.Hi - 1);
                const int ix = min(max(ox * p.sw - p.pl + (t % 3) * p.dw, 0), p.Wi - 1);
                ip[t] = base + (size_t)iy * p.Wi + ix;
            }
            size_t ifirst = ip[0];
#pragma unroll
            for (int t = 1; t < 9; ++t) ifirst = first == t ? ip[t] : ifirst;
#pragma unroll
            for (int t = 0; t < 9; ++t) x[u][t] = vload<T, N>(in + (((tp[u] >> t) & 1) ? ip[t] : ifirst) * C + c);
            if (ACT >= 0)
                load_state<T, 1>(q[u], tr[u], valid[u], (size_t)pix[u], gl, G, C, (const T *)epi.prev, (const T *)epi.trunc);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k + u * ppi >= n) continue;  // wave-uniform
            float acc[N];
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] = 0.f;
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const Vec<T, N> xs = vkeep<T, N>(x[u][t], (tp[u] >> t) & 1);
                const Vec<T, N> wt = LW ? s_w[LW ? t : 0][c / N] : w[LW ? 0 : t];
#pragma unroll
                for (int e = 0; e < N; ++e) acc[e] = __builtin_fmaf(float(xs.v[e]), float(wt.v[e]), acc[e]);
            }
            Vec<T, N> dl[1];
            if (bias != nullptr) {
#pragma unroll
                for (int e = 0; e < N; ++e) acc[e] += float(bv.v[e]);
            }
#pragma unroll
            for (int e = 0; e < N; ++e) dl[0].v[e] = T(acc[e]);
            if (ACT < 0) {
                if (valid[u]) vstore<T, N>(out + (size_t)pix[u] * C + c, dl[0]);
            } else {
                act_trunc_pixel<T, 1, (ACT < 0 ? 0 : ACT)>(dl, q[u], tr[u], valid[u], (size_t)pix[u], gl, G, C, out,
                                                            (T *)epi.prev, (T *)epi.trunc, out_mask, T(epi.thr), epi.mode);
            }
        }
    }
}

// ------------------------------------------------------------------ few input channels
// Network stems (RGB input): groups == 1, Cin <= 4.  Same one-group-per-output-pixel shape as
// the depthwise kernel; a lane owns N consecutive output channels, input values are scalar
// broadcasts.  fp16 filters are read in the reference layout directly: for an even channel
// offset the even outputs sit in row ci and the odd ones in row ci ^ 1 of the swizzle.
// K3 (3x3): the filter is staged once per workgroup into LDS in [tap][ci][co] order (un-swizzled)
// and the 9 x Cin input values and the cached state are requested before the mask words have
// arrived, so the kernel is one memory round trip instead of one per active tap.
template <typename T, int ACT, bool K3>
__global__ void __launch_bounds__(256)
conv_fewcin_kernel(ConvP p, const T *__restrict__ in, const T *__restrict__ filter,
                   const T *__restrict__ bias, T *__restrict__ out,
                   const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, EpiP epi,
                   int lg, int staged) {
    constexpr int N = Vec16<T>::N;
    constexpr int MAXCI = 4;
    const int G = 1 << lg;
    const int C = p.Co;
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int po = gid >> lg, gl = gid & (G - 1);
    const int P_out = p.B * p.Ho * p.Wo;
    const bool valid = po < P_out;
    const int b = po / (p.Ho * p.Wo);
    const int r = po - b * p.Ho * p.Wo;
    const int oy = r / p.Wo, ox = r - oy * p.Wo;
    const int K2 = p.Kh * p.Kw;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const int glo = lane_id() & ~(G - 1);
    const uint64_t gmask = G >= WAVE ? ~0ull : ((1ull << G) - 1ull);

    extern __shared__ __align__(16) unsigned char s_raw[];
    T *s_w = reinterpret_cast<T *>(s_raw);
    float xin[K3 ? 9 : 1][MAXCI];
    Vec<T, N> q[1], tr[1];
    if (K3 || staged) {  // the filter, un-swizzled, in [tap][ci][co] order
        const int cv = C / N;  // 16-byte vectors per filter row (C % N == 0, so w_co == C)
        const int total = K2 * p.Ci * cv;
        for (int i = threadIdx.x; i < total; i += blockDim.x) {
            const int v = i % cv, r2 = i / cv;
            const int ci = r2 % p.Ci, t = r2 / p.Ci;
            Vec<T, N> w = vload<T, N>(filter + ((size_t)ci * K2 + t) * p.w_co + v * N);
            if (p.swz) {  // odd output channels live in the partner row of the pair swizzle
                const Vec<T, N> w1 = vload<T, N>(filter + ((size_t)(ci ^ 1) * K2 + t) * p.w_co + v * N);
#pragma unroll
                for (int j = 1; j < N; j += 2) w.v[j] = w1.v[j];
            }
            vstore<T, N>(s_w + (size_t)i * N, w);
        }
    }
    if (K3) {
        const int pc = valid ? po : 0;
        const int cb = pc / (p.Ho * p.Wo), cr = pc - cb * p.Ho * p.Wo;
        const int cy = cr / p.Wo, cx = cr - cy * p.Wo;
        const T *inb = in + (size_t)cb * p.Hi * p.Wi * p.Ci;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int ky = t / 3, kx = t - ky * 3;
            const int iy = min(max(cy * p.sh - p.pt + ky * p.dh, 0), p.Hi - 1);
            const int ix = min(max(cx * p.sw - p.pl + kx * p.dw, 0), p.Wi - 1);
            const T *xr = inb + (size_t)(iy * p.Wi + ix) * p.Ci;
#pragma unroll
            for (int ci = 0; ci < MAXCI; ++ci) xin[t][ci] = float(xr[min(ci, p.Ci - 1)]);
        }
        if (ACT >= 0) {
            const int cc = min(gl * N, C - N);
            q[0] = vload<T, N>((const T *)epi.prev + (size_t)pc * C + cc);
            tr[0] = vload<T, N>((const T *)epi.trunc + (size_t)pc * C + cc);
        }
    }
    if (K3 || staged) __syncthreads();

    uint64_t taps = 0;
    for (int j = 0; j < K2; j += G) {
        const int t = j + gl;
        bool m = false;
        if (valid && t < K2) {
            const int ky = t / p.Kw, kx = t - ky * p.Kw;
            const int iy = oy * p.sh - p.pt + ky * p.dh, ix = ox * p.sw - p.pl + kx * p.dw;
            if (iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi) m = mb[iy * p.Wi + ix] != 0;
        }
        taps |= ((ballot(m) >> glo) & gmask) << j;
    }
    const bool active = valid && taps != 0;
    if (valid && gl == 0) out_mask[po] = active ? 1 : 0;
    if (ballot(active) == 0) return;

    const int c = gl * N;
    const bool lane_on = active && c < C;
    if (ACT >= 0 && !K3)
        load_state<T, 1>(q, tr, active, (size_t)po, gl, G, C, (const T *)epi.prev, (const T *)epi.trunc);
    float acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = 0.f;
    if (K3) {
        if (lane_on) {
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const bool on = (taps >> t) & 1ull;
#pragma unroll
                for (int ci = 0; ci < MAXCI; ++ci) {
                    if (ci >= p.Ci) break;
                    const float xv = on ? xin[t][ci] : 0.f;
                    const Vec<T, N> w = vload<T, N>(s_w + (size_t)(t * p.Ci + ci) * C + c);
#pragma unroll
                    for (int j = 0; j < N; ++j) acc[j] = __builtin_fmaf(xv, float(w.v[j]), acc[j]);
                }
            }
        }
    } else if (staged) {
        // any kernel size with the filter in LDS: the inputs of up to seven taps of a filter row
        // are requested together from clamped addresses and zero-selected afterwards
        if (lane_on) {
            constexpr int RW = 7;
            const T *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
            for (int ky = 0; ky < p.Kh; ++ky) {
                const int iy = min(max(oy * p.sh - p.pt + ky * p.dh, 0), p.Hi - 1);
                for (int kx0 = 0; kx0 < p.Kw; kx0 += RW) {
                    float xr[RW][MAXCI];
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        const int ix = min(max(ox * p.sw - p.pl + min(kx0 + u, p.Kw - 1) * p.dw, 0), p.Wi - 1);
                        const T *xp = inb + (size_t)(iy * p.Wi + ix) * p.Ci;
#pragma unroll
                        for (int ci = 0; ci < MAXCI; ++ci) xr[u][ci] = float(xp[min(ci, p.Ci - 1)]);
                    }
#pragma unroll
                    for (int u = 0; u < RW; ++u) {
                        if (kx0 + u >= p.Kw) break;  // uniform
                        const int t = ky * p.Kw + kx0 + u;
                        const bool on = (taps >> t) & 1ull;
#pragma unroll
                        for (int ci = 0; ci < MAXCI; ++ci) {
                            if (ci >= p.Ci) break;
                            const float xv = on ? xr[u][ci] : 0.f;
                            const Vec<T, N> w = vload<T, N>(s_w + (size_t)(t * p.Ci + ci) * C + c);
#pragma unroll
                            for (int j = 0; j < N; ++j) acc[j] = __builtin_fmaf(xv, float(w.v[j]), acc[j]);
                        }
                    }
                }
            }
        }
    } else if (lane_on) {
        const T *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
        for (int t = 0; t < K2; ++t) {
            if (!((taps >> t) & 1ull)) continue;
            const int ky = t / p.Kw, kx = t - ky * p.Kw;
            const int iy = oy * p.sh - p.pt + ky * p.dh, ix = ox * p.sw - p.pl + kx * p.dw;
            const T *xr = inb + (size_t)(iy * p.Wi + ix) * p.Ci;
#pragma unroll
            for (int ci = 0; ci < MAXCI; ++ci) {
                if (ci >= p.Ci) break;
                const float xv = float(xr[ci]);
                Vec<T, N> w = vload<T, N>(filter + ((size_t)ci * K2 + t) * p.w_co + c);
                if (p.swz) {
                    const Vec<T, N> w1 = vload<T, N>(filter + ((size_t)(ci ^ 1) * K2 + t) * p.w_co + c);
#pragma unroll
                    for (int j = 1; j < N; j += 2) w.v[j] = w1.v[j];
                }
#pragma unroll
                for (int j = 0; j < N; ++j) acc[j] = __builtin_fmaf(xv, float(w.v[j]), acc[j]);
            }
        }
    }
    Vec<T, N> dl[1];
    if (lane_on) {
        if (bias != nullptr) {
            const Vec<T, N> bv = vload<T, N>(bias + c);
#pragma unroll
            for (int j = 0; j < N; ++j) acc[j] += float(bv.v[j]);
        }
#pragma unroll
        for (int j = 0; j < N; ++j) dl[0].v[j] = T(acc[j]);
    }
    if (ACT < 0) {
        if (lane_on) vstore<T, N>(out + (size_t)po * C + c, dl[0]);
    } else {
        act_trunc_pixel<T, 1, (ACT < 0 ? 0 : ACT)>(dl, q, tr, active, (size_t)po, gl, G, C, out,
                                                     (T *)epi.prev, (T *)epi.trunc, out_mask,
                                                     T(epi.thr), epi.mode);
    }
}

// ------------------------------------------------------------------------------------ MFMA
// Implicit GEMM on v_mfma_f32_16x16x32_f16 for any kernel size / stride / dilation and for the
// transposed convolution: rows = 16 output channels (packed filter, fragment order), columns =
// 16 compacted output pixels of the 8x8 tile, reduction over (tap, input channel) in steps of
// 32, step index s = tap * ksteps + channel step (the packed filter is linear in s).
//
//   * the mask phase also builds a table in LDS: for every (tap, compacted pixel) the index of
//     the input pixel it reads, or -1 if that input is out of bounds or inactive; taps that no
//     pixel of the tile uses are skipped altogether;
//   * a wavefront accumulates R channel tiles x 4 pixel tiles, so a reduction step costs
//     R + 4 fragment loads for 4 * R MFMAs; the KW wavefronts of a workgroup split the steps
//     round-robin and their partial sums meet in LDS (added in ascending wavefront order);
//   * all fragment loads of S steps are issued unconditionally (clamped addresses) before the
//     first MFMA of the chunk; input fragments of invalid (tap, pixel) pairs are zeroed by
//     selection afterwards -- unlike the pointwise case they would reach valid outputs.
constexpr int MFMA_MAX_TAPS = 64;

template <typename E, bool TR, int KW, int R, int S>
__global__ void __launch_bounds__(KW * WAVE)
conv_mfma_kernel(ConvP p, const E *__restrict__ in, const E *__restrict__ wp,
                 const E *__restrict__ bias, E *__restrict__ out,
                 const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, int co_blocks,
                 int ci_p) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NT = 4;
    __shared__ int s_list[TILE_PX];
    __shared__ int s_n;
    __shared__ int s_src[MFMA_MAX_TAPS * TILE_PX];
    __shared__ int s_taplist[MFMA_MAX_TAPS];
    __shared__ int s_ntaps;
    __shared__ float4_t s_red[KW > 1 ? KW * NT * WAVE : 1];
    const int b = blockIdx.z / co_blocks;
    const int cb = blockIdx.z % co_blocks;
    // transposed: blockIdx = (tile, stride phase) interleaved, pixels of a tile one stride apart
    const int ys = TR ? p.sh : 1, xs = TR ? p.sw : 1;
    const int ty0 = (blockIdx.y / ys) * TILE * ys + blockIdx.y % ys;
    const int tx0 = (blockIdx.x / xs) * TILE * xs + blockIdx.x % xs;
    const int n = tile_front<TR>(p, mask, out_mask, b, ty0, tx0, ys, xs, cb == 0, s_list, s_src,
                                 s_taplist, &s_ntaps, &s_n);
    if (n == 0) return;

    const int kw = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;  // row / column inside a tile, k-quarter
    const int K2 = p.Kh * p.Kw;
    const int n_tiles = (n + 15) >> 4;
    const int co_tiles = (p.Co + 15) >> 4;
    const E *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;

    float4_t acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[r][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int ksteps = ci_p >> 5;
    const int total = s_ntaps * ksteps;  // steps over the taps in use only
    const E *wfrag[R];
#pragma unroll
    for (int r = 0; r < R; ++r)  // surplus channel tiles re-read the last one and are not stored
        wfrag[r] = wp + (size_t)min(cb * R + r, co_tiles - 1) * K2 * ksteps * 512 + lane * 8;

    for (int s0 = kw; s0 < total; s0 += S * KW) {
        E8 a[S][R], x[S][NT];
        int src[S][NT];
        bool use[S];
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int s = min(s0 + i * KW, total - 1);
            const int ti = s / ksteps, ks = s - ti * ksteps;
            const int tap = s_taplist[ti];
            const int k = min((ks << 5) + kq * 8, p.Ci - 8);
            use[i] = s0 + i * KW < total;  // wave-uniform
#pragma unroll
            for (int r = 0; r < R; ++r)
                a[i][r] = *reinterpret_cast<const E8 *>(wfrag[r] + (size_t)(tap * ksteps + ks) * 512);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                src[i][nt] = s_src[(tap << 6) + nt * 16 + l16];
                x[i][nt] = *reinterpret_cast<const E8 *>(inb + (size_t)max(src[i][nt], 0) * p.Ci + k);
            }
        }
#pragma unroll
        for (int i = 0; i < S; ++i) {
            if (!use[i]) continue;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (nt >= n_tiles) continue;  // wave-uniform
                const E8 xz = keep8(x[i][nt], src[i][nt] >= 0);
#pragma unroll
                for (int r = 0; r < R; ++r)
                    acc[r][nt] = Elem16<E>::mfma(a[i][r], xz, acc[r][nt]);
            }
        }
    }

    // wavefront kw finishes pixel tiles kw, kw + KW, ... of every channel tile
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (KW > 1) {
            if (r > 0) __syncthreads();
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) s_red[(kw * NT + nt) * WAVE + lane] = acc[r][nt];
            __syncthreads();
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if ((nt % KW) != kw) continue;
                float4_t sum = s_red[nt * WAVE + lane];
#pragma unroll
                for (int q = 1; q < KW; ++q) sum += s_red[(q * NT + nt) * WAVE + lane];
                acc[r][nt] = sum;
            }
        }
        const int ct = cb * R + r;
        if (ct >= co_tiles) continue;
        // lane holds channels ct*16 + kq*4 + {0..3} of pixel (nt, l16)
        const int co = ct * 16 + kq * 4;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias != nullptr) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (co + i < p.Co) bv[i] = float(bias[co + i]);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if ((nt % KW) != kw && KW > 1) continue;
            const int pix = nt * 16 + l16;
            if (pix >= n) continue;
            const int code = s_list[pix];
            E *o = out + (((size_t)b * p.Ho + (code >> 16)) * p.Wo + (code & 0xffff)) * p.Co + co;
            if (co + 3 < p.Co && (p.Co & 3) == 0) {
                E4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = E(acc[r][nt][i] + bv[i]);
                *reinterpret_cast<E4 *>(o) = v;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (co + i < p.Co) o[i] = E(acc[r][nt][i] + bv[i]);
            }
        }
    }
}

// Larger layers: the input window ("halo") of an 8x8 output tile is staged in LDS once and the
// input fragments of every tap are read from there, so global traffic per workgroup is the halo
// plus the filter fragments.  Inactive and out-of-bounds halo pixels are staged as zeros, which
// removes every per-fragment validity test from the reduction loop.
//   * the wavefronts of a workgroup split the output channels (R tiles of 16 each) and, KS-fold,
//     the reduction steps; all accumulate the same (up to four) compacted 16-pixel tiles.  An
//     input fragment read from LDS feeds R MFMAs, so R = 2 with the steps split over two
//     wavefronts moves half the LDS bytes of R = 1 with four channel groups at the same number
//     of wavefronts (measured: 3 to 15 % faster, most for long reductions); the partial sums
//     of the slices meet in LDS, added in ascending slice order;
//   * the halo is staged in chunks of `kcc` reduction steps (32 channels each) sized to the LDS
//     budget; a pixel row is padded by 16 bytes so that neighbouring pixels start in different
//     banks;
//   * filter fragments (contiguous 1 KB reads) stream through a ring of D register buffers of
//     S steps each, so D - 1 chunks are in flight while one is consumed: 4 LDS reads and
//     4 * R MFMAs per step.
// Operands of a DCAdd fused behind a convolution: a = residual, b = convolution.
template <typename E>
struct PatchRes {  // DCAdd fused behind the convolution: a = residual, b = convolution
    const E *values;
    const int32_t *mask;
    E *prev;
    float wa, wb;
    int act;
};

constexpr int LDS_MAX_HALO = 1024;
constexpr int LDS_MAX_STEPS = 1024;

// The layer's activation / truncation finished in the convolution's launch (FIN), for layers whose
// workgroups hold all output channels of their pixels (the keep decision of a pixel needs them
// all): the wavefronts put their rounded sums into LDS as pixel rows and the workgroup runs
// act_trunc_pixel over the rows, 2^lg lanes per pixel; the cached state of the first pass is
// requested before the reduction.  `out` receives the activated differences of the kept pixels
// only.  Offered where the launch has at most one workgroup per compute unit: the finishing stores
// three tensors, which a workgroup that is followed by another on its compute unit only delays
// (measured on 64 -> 64 at 136 x 240, 510 workgroups: 8.3 + 4.6 us as two launches, 13.5 us as
// one; 128 -> 64 at 68 x 120, 135 workgroups: 7.7 + 2.9 -> 9.1 us).
template <typename E>
struct LdsFin {
    E *prev, *trunc;
    float thr;
    int mode, act;
    int lg, iters;  // 2^lg lanes per pixel, `iters` 16-byte vectors per lane
};

// The finishing passes: 2^lg lanes per pixel over the compacted list `list` of `n` tile pixels
// (`opix`: tile pixel -> pixel index in the output map).  The sums lie in LDS, row `slot` at
// rows + slot * row_b; q0 / tr0 hold the state of the first pass.
template <typename E, int ITERS, int ACT, typename PixelOf>
__device__ __forceinline__ void lds_finish(const LdsFin<E> &f, const int *list, int n, int tid, int nthr, int Co,
                                           E *__restrict__ out, int32_t *__restrict__ out_mask, PixelOf opix,
                                           const unsigned char *rows, int row_b,
                                           const Vec<E, Vec16<E>::N> (&q0)[2], const Vec<E, Vec16<E>::N> (&tr0)[2]) {
    constexpr int N = Vec16<E>::N;
    const int G = 1 << f.lg, gl = tid & (G - 1), groups = nthr >> f.lg;
    for (int s0 = 0; s0 < n; s0 += groups) {  // the same number of passes in every wavefront
        const int slot = min(s0 + (tid >> f.lg), n - 1);
        const bool valid = s0 + (tid >> f.lg) < n;
        const size_t px = opix(list[slot] & 63);
        Vec<E, N> dl[ITERS], q[ITERS], tr[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {  // later passes request their state here
            const int c = min((it * G + gl) * N, Co - N);
            const size_t off = px * Co + c;
            dl[it] = *reinterpret_cast<const Vec<E, N> *>(rows + slot * row_b + c * (int)sizeof(E));
            if (s0 == 0) {
                q[it] = q0[it];
                tr[it] = tr0[it];
            } else {
                q[it] = vload<E, N>(f.prev + off);
                tr[it] = vload<E, N>(f.trunc + off);
            }
        }
        const bool keep = act_trunc_pixel<E, ITERS, ACT>(dl, q, tr, valid, px, gl, G, Co, out, f.prev, f.trunc,
                                                         out_mask, E(f.thr), f.mode);
        if (valid && keep && gl == 0) out_mask[px] = 1;
    }
}

template <typename E, int R, int S, int D, int KS, bool TR, bool ADD, bool FIN = false>
__global__ void __launch_bounds__(8 * WAVE)
conv_lds_mfma_kernel(ConvP p, const E *__restrict__ in, const E *__restrict__ wp,
                     const E *__restrict__ bias, E *__restrict__ out,
                     const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                     int co_blocks, int ci_p, int hal_h, int hal_w, int kcc, int lgv, PatchRes<E> rs,
                     LdsFin<E> fin_args) {
    static_assert(!(FIN && (TR || ADD)), "the finishing pass exists for plain convolutions");
    // FIN: launched with co_blocks == 1
    // ADD: the sum of a DCAdd without activation rides on the accumulators.  (With an activation the
    // accumulated sum has to be read and written as well; in this kernel's 8-byte-per-lane epilogue
    // that costs what the separate add kernel costs -- measured -- so that form is not offered.)
    // ADD && TR: a transposed convolution whose every stride phase has taps (window >= stride).
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr int NT = 4;
    constexpr int TPW = R * NT / KS;  // output tiles of 16 x 16 a wavefront finishes
    static_assert(TPW * KS == R * NT, "the reduction slices of a channel group share its tiles evenly");
    extern __shared__ __align__(16) unsigned char s_halo[];
    __shared__ int s_hpix[LDS_MAX_HALO];
    __shared__ int2 s_step[LDS_MAX_STEPS];
    // compacted tile pixels (index | 64 if updated | 128 if the residual is), one copy per wavefront:
    // every wavefront dilates and compacts the mask itself
    __shared__ int s_list[8][TILE_PX];
    const int b = blockIdx.z / co_blocks, cb = blockIdx.z % co_blocks;
    // TR (transposed, dilation 1): the outputs of one stride phase (py, px) form an ordinary
    // convolution of the input with the A x Bt filter taps ky = ry + a * stride, kx = rx + b * stride:
    // out[(J * sh + py), (I * sw + px)] = sum_ab W[ky][kx] * in[J + qy - a][I + qx - b].  A tile is
    // 8 x 8 such outputs (J, I); blockIdx = (tile, phase) interleaved.
    const int ys = TR ? p.sh : 1, xs = TR ? p.sw : 1;
    const int phy = blockIdx.y % ys, phx = blockIdx.x % xs;
    const int ty0 = (blockIdx.y / ys) * TILE, tx0 = (blockIdx.x / xs) * TILE;
    const int ry = TR ? (phy + p.pt) % p.sh : 0, rx = TR ? (phx + p.pl) % p.sw : 0;
    const int A = TR ? (p.Kh - ry + p.sh - 1) / p.sh : p.Kh;   // taps of this tile per dimension
    const int Bt = TR ? (p.Kw - rx + p.sw - 1) / p.sw : p.Kw;
    const int Amax = (p.Kh + p.sh - 1) / p.sh, Bmax = (p.Kw + p.sw - 1) / p.sw;
    const int VK2 = A * Bt;
    // output coordinate of tile pixel (ly, lx); halo step per output step
    auto out_y = [&](int ly) { return TR ? (ty0 + ly) * ys + phy : ty0 + ly; };
    auto out_x = [&](int lx) { return TR ? (tx0 + lx) * xs + phx : tx0 + lx; };
    const int vsy = TR ? 1 : p.sh, vsx = TR ? 1 : p.sw;
    // halo element offset of tap (a, b2) relative to an output's halo origin
    auto tap_off = [&](int a, int b2) {
        return TR ? (Amax - 1 - a) * hal_w + (Bmax - 1 - b2) : a * p.dh * hal_w + b2 * p.dw;
    };
    const int tid = threadIdx.x, nthr = blockDim.x, nw = nthr / WAVE;
    const int wv = wave_id(), lane = lane_id();
    // wavefront = (channel group cw, reduction slice kz): slice kz takes steps kz, kz + KS, ...
    const int ncw = nw / KS, cw = wv % ncw, kz = wv / ncw;
    const int l16 = lane & 15, kq = lane >> 4;
    const int hpx = hal_h * hal_w;
    const int iy0 = TR ? ty0 + (phy + p.pt - ry) / p.sh - (Amax - 1) : ty0 * p.sh - p.pt;
    const int ix0 = TR ? tx0 + (phx + p.pl - rx) / p.sw - (Bmax - 1) : tx0 * p.sw - p.pl;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const int co_tiles = (p.Co + 15) >> 4;
    const int ksteps = ci_p >> 5;
    const int K2 = p.Kh * p.Kw;
    const int row = kcc * 64 + 16;  // bytes per staged halo pixel

    // Step table of a channel chunk: for reduction step j = tap * kcur + ks the LDS byte offset of
    // its input fragment relative to a pixel's halo origin, and its fragment offset in the
    // packed filter.  Entries past the last step repeat it (their products are zeroed).
    auto build_steps = [&](int kbase, int kcur) {
        const int nsteps = VK2 * kcur;
        const int padded = (nsteps + S * D * KS - 1) / (S * D * KS) * (S * D * KS);
        for (int j = tid; j < padded; j += nthr) {
            const int jj = min(j, nsteps - 1);
            const int tap = jj / kcur, ks = jj - tap * kcur;
            const int ta = tap / Bt, tb = tap - ta * Bt;
            const int real = TR ? (ry + ta * p.sh) * p.Kw + rx + tb * p.sw : tap;  // tap of the filter
            s_step[j] = int2{tap_off(ta, tb) * row + ks * 64, (real * ksteps + kbase + ks) * 512};
        }
    };
    if (TR && VK2 == 0) {  // a phase without taps (kernel smaller than the stride): nothing updated
        if (cb == 0 && tid < WAVE) {
            const int oy = out_y(tid >> 3), ox = out_x(tid & 7);
            if (oy < p.Ho && ox < p.Wo) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = 0;
        }
        return;
    }
    // Front end.  Nothing in it waits for anything it does not need: the mask word of halo pixel
    // `tid` and the halo ROWS of this lane's staging slots are requested first, the rows from
    // addresses that follow from the tile's coordinates alone (what an inactive pixel returns is
    // zeroed when it is stored); the step table is built while they travel; the filter chunks are
    // requested behind the rows, so that the rows are not queued behind them.
    auto halo_pixel = [&](int i, bool &ok) {  // position in the input map (clamped into it), and whether it lies inside
        const int hy = i / hal_w, hx = i - hy * hal_w;
        const int iy = iy0 + hy, ix = ix0 + hx;
        ok = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
        return min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1);
    };
    bool ok0;
    const int hpix0 = halo_pixel(min(tid, hpx - 1), ok0);
    const int hword0 = mb[hpix0];
    // Staging of channels [kbase * 32, (kbase + kcur) * 32) of the halo: 2^lgv lanes per pixel, SU
    // pixels per lane in flight (a 10 x 10 halo is one pass); inactive pixels are stored as zeros.
    constexpr int SU = 8;
    const E *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
    const int sv = tid & ((1 << lgv) - 1), hstep = nthr >> lgv;
    E8 val0[SU];
    {
        const int c = min(sv * 8, p.Ci - 8);
        // slot u of this lane lies hstep halo pixels behind slot u - 1: row and column follow from
        // one division
        const int dy = hstep / hal_w, dx = hstep - dy * hal_w;  // uniform
        int hy = (tid >> lgv) / hal_w, hx = (tid >> lgv) - hy * hal_w;
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const bool in_halo = hy < hal_h;  // past the halo: the last pixel again, not stored
            const int iy = iy0 + (in_halo ? hy : hal_h - 1), ix = ix0 + (in_halo ? hx : hal_w - 1);
            const int px = min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1);
            val0[u] = *reinterpret_cast<const E8 *>(inb + (size_t)px * p.Ci + c);
            hx += dx;
            hy += dy;
            if (hx >= hal_w) {
                hx -= hal_w;
                ++hy;
            }
        }
    }
    // the tile pixel of this lane (every wavefront dilates the mask for all 64 pixels itself)
    const int ly = lane >> 3, lx = lane & 7;
    const int oy = out_y(ly), ox = out_x(lx);
    const bool inside = oy < p.Ho && ox < p.Wo;
    int rword = 0;  // ADD: the residual's mask word
    if (ADD) rword = rs.mask[((size_t)b * p.Ho + min(oy, p.Ho - 1)) * p.Wo + min(ox, p.Wo - 1)];
    build_steps(0, min(kcc, ksteps));
    // mask words -> pixel table: global pixel index of every active in-bounds halo pixel, else -1
    if (tid < hpx) s_hpix[tid] = (ok0 && hword0 != 0) ? hpix0 : -1;
    for (int i = tid + nthr; i < hpx; i += nthr) {
        bool ok;
        const int px = halo_pixel(i, ok);
        const int word = mb[px];
        s_hpix[i] = (ok && word != 0) ? px : -1;
    }
    __syncthreads();

    // Filter fragments stream through a ring of D register buffers of S steps each, so D - 1
    // chunks are in flight while one is consumed.  The first D chunks are requested here, before
    // the mask phase and the staging, whose latencies they overlap.
    unsigned wfrag[R];  // element offset of the wavefront's channel tiles in the packed filter
#pragma unroll
    for (int r = 0; r < R; ++r)  // surplus channel tiles re-read the last one and are not stored
        wfrag[r] = (unsigned)min((cb * ncw + cw) * R + r, co_tiles - 1) * K2 * ksteps * 512 + lane * 8;
    E8 a[D][S][R];
    int xo[D][S];
    int jl = 0;
    auto load_chunk = [&](E8 (&ac)[S][R], int (&xc)[S]) {
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int2 e = s_step[(jl + i) * KS + kz];
            xc[i] = e.x;
#pragma unroll
            for (int r = 0; r < R; ++r)
                ac[i][r] = *reinterpret_cast<const E8 *>(wp + (wfrag[r] + (unsigned)e.y));
        }
        jl += S;
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load_chunk(a[d], xo[d]);
    // bias of the lane's four channels for the tiles this wavefront finishes: tiles
    // [kz * TPW, (kz + 1) * TPW) of its channel group, tile t = (channel tile t / NT, pixel tile t % NT)
    // (the TPW tiles lie in BR channel tiles: all R of them without reduction slices, else one)
    constexpr int BR = TPW > NT ? TPW / NT : 1;
    E bv[BR][4];
#pragma unroll
    for (int q = 0; q < BR; ++q) {
        const int co = ((cb * ncw + cw) * R + (kz * TPW) / NT + q) * 16 + kq * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) bv[q][i] = bias != nullptr ? bias[min(co + i, p.Co - 1)] : E(0);
    }
    auto stage_load = [&](int kbase, int h0, E8 (&val)[SU], int (&px)[SU]) {
        const int c = min((kbase << 5) + sv * 8, p.Ci - 8);
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            px[u] = s_hpix[min(h0 + u * hstep, hpx - 1)];
            val[u] = *reinterpret_cast<const E8 *>(inb + (size_t)max(px[u], 0) * p.Ci + c);
        }
    };
    auto stage_store = [&](int kbase, int kcur, int h0, const E8 (&val)[SU], const int (&px)[SU]) {
        const bool vok = sv < kcur * 4 && (kbase << 5) + sv * 8 < p.Ci;
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const int hp = h0 + u * hstep;
            if (hp < hpx && sv < kcur * 4)
                *reinterpret_cast<E8 *>(s_halo + hp * row + sv * 16) = keep8(val[u], vok && px[u] >= 0);
        }
    };

    // dilate the mask over the window and compact the updated pixels: by every wavefront for itself
    // (the same table, hence the same list in all of them), while the halo rows are still travelling
    int n;
    bool tile_upd, any_px;
    {
        bool upd = false;
        const int base = ly * vsy * hal_w + lx * vsx;
        if (!TR && p.Kh == 3 && p.Kw == 3) {  // the common window: nine independent reads
#pragma unroll
            for (int t = 0; t < 9; ++t) upd |= s_hpix[base + (t / 3) * p.dh * hal_w + (t % 3) * p.dw] >= 0;
        } else {
            for (int ta = 0; ta < A; ++ta)
                for (int tb = 0; tb < Bt; ++tb) upd |= s_hpix[base + tap_off(ta, tb)] >= 0;
        }
        upd = upd && inside;
        const bool radd = ADD && inside && rword != 0;
        const bool any = upd || radd;  // ADD: the union of both masks is written and compacted
        any_px = any;
        // FIN: the finishing workgroup writes the mask; a tile without updates has none
        const int rank = wave_rank(any, n);
        if (inside && cb == 0 && wv == 0 && (!FIN || n == 0))
            out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = any ? 1 : 0;
        if (any) s_list[wv][rank] = lane | (upd ? 64 : 0) | (radd ? 128 : 0);
        tile_upd = ballot(upd) != 0;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if (n == 0) return;  // the same in every wavefront
    {   // the rows requested at the start: into LDS, those of inactive pixels as zeros
        int px0[SU];
#pragma unroll
        for (int u = 0; u < SU; ++u) px0[u] = s_hpix[min((tid >> lgv) + u * hstep, hpx - 1)];
        stage_store(0, min(kcc, ksteps), tid >> lgv, val0, px0);
    }
    __syncthreads();

    const int n_tiles = (n + 15) >> 4;
    int hbase[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int slot = nt * 16 + l16;
        const int loc = slot < n ? (s_list[wv][slot] & 63) : 0;
        hbase[nt] = ((loc >> 3) * vsy * hal_w + (loc & 7) * vsx) * row + kq * 16;
    }
    // ADD: the operands of the sum for the tiles this wavefront finishes, requested before the
    // reduction, which they overlap
    E4 rv[ADD ? TPW : 1];
    if (ADD) {
#pragma unroll
        for (int q = 0; q < TPW; ++q) {
            const int t = kz * TPW + q, nt = t % NT;
            const int co = ((cb * ncw + cw) * R + t / NT) * 16 + kq * 4;
            const bool vec = co + 3 < p.Co && (p.Co & 3) == 0;
            rv[q] = zero4<E>();
            const int pix = nt * 16 + l16;
            if (pix >= n || co >= p.Co) continue;
            const int code = s_list[wv][pix], loc = code & 63;
            const size_t off = (((size_t)b * p.Ho + out_y(loc >> 3)) * p.Wo + out_x(loc & 7)) * p.Co;
            const bool radd = (code & 128) != 0;
            if (vec) {
                if (radd) rv[q] = *reinterpret_cast<const E4 *>(rs.values + off + co);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int c = min(co + i, p.Co - 1);
                    if (radd) rv[q][i] = rs.values[off + c];
                }
            }
        }
    }
    // FIN, all channels in this workgroup: the cached state of the first finishing pass, requested
    // before the reduction, which it overlaps
    auto opix = [&](int loc) { return ((size_t)b * p.Ho + out_y(loc >> 3)) * p.Wo + out_x(loc & 7); };
    Vec<E, Vec16<E>::N> fq[2], ftr[2];
    if (FIN) {
        const int slot = min(tid >> fin_args.lg, n - 1), gl = tid & ((1 << fin_args.lg) - 1);
        const size_t row = opix(s_list[wv][slot] & 63) * p.Co;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            if (it < fin_args.iters) {
                const int c = min(((it << fin_args.lg) + gl) * 8, p.Co - 8);
                fq[it] = vload<E, 8>(fin_args.prev + row + c);
                ftr[it] = vload<E, 8>(fin_args.trunc + row + c);
            }
        }
    }
    float4_t acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[r][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ADD: a tile reached by the residual only has nothing to contract (uniform)
    const int kend = (ADD && !tile_upd) ? 0 : ksteps;
    for (int kbase = 0; kbase < kend; kbase += kcc) {
        const int kcur = min(kcc, ksteps - kbase);
        if (kbase > 0) {
            __syncthreads();
            build_steps(kbase, kcur);
        }
        // remaining staging passes (all of them for the channel chunks after the first)
        for (int h0 = (tid >> lgv) + (kbase == 0 ? SU * hstep : 0); h0 < hpx; h0 += SU * hstep) {
            E8 val[SU];
            int px[SU];
            stage_load(kbase, h0, val, px);
            stage_store(kbase, kcur, h0, val, px);
        }
        if (kbase > 0 || hpx > SU * hstep) __syncthreads();  // uniform: something was staged here
        const int nsteps = VK2 * kcur;
        const int groups = (nsteps + S * D * KS - 1) / (S * D * KS);  // of D chunks of S steps per slice
        if (kbase > 0) {
            jl = 0;
#pragma unroll
            for (int d = 0; d < D; ++d) load_chunk(a[d], xo[d]);
        }
        // All groups but the last are complete and run without any test; NTA (number of 16-pixel
        // tiles in use) is a compile-time constant, so the loop body is one branch-free block.
        auto reduce = [&](auto nta_tag) {
            constexpr int NTA = decltype(nta_tag)::value;
            // input fragments are read from LDS one step ahead of the MFMAs that consume them
            E8 xq[NTA];
            auto read_x = [&](E8 (&x)[NTA], int off) {
#pragma unroll
                for (int nt = 0; nt < NTA; ++nt)
                    x[nt] = *reinterpret_cast<const E8 *>(s_halo + hbase[nt] + off);
            };
            auto compute_chunk = [&](const E8 (&ac)[S][R], const int (&xc)[S], int next_off, auto tail_tag, int j0) {
#pragma unroll
                for (int i = 0; i < S; ++i) {
                    E8 xn[NTA];
                    read_x(xn, i + 1 < S ? xc[i + 1] : next_off);
#pragma unroll
                    for (int nt = 0; nt < NTA; ++nt) {
                        if (decltype(tail_tag)::value) xq[nt] = keep8(xq[nt], (j0 + i) * KS + kz < nsteps);
#pragma unroll
                        for (int r = 0; r < R; ++r)
                            acc[r][nt] = Elem16<E>::mfma(ac[i][r], xq[nt], acc[r][nt]);
                    }
#pragma unroll
                    for (int nt = 0; nt < NTA; ++nt) xq[nt] = xn[nt];
                }
            };
            read_x(xq, xo[0][0]);
            for (int g = 0; g + 1 < groups; ++g) {
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    // the chunk after the last one of the ring is the first of the next group,
                    // already reloaded below
                    compute_chunk(a[d], xo[d], xo[(d + 1) % D][0], std::false_type{}, 0);
                    load_chunk(a[d], xo[d]);
                    // the refill stays here, D - 1 chunks ahead of its use: left to itself the
                    // scheduler gathers the requests of all chunks at the end of the iteration,
                    // where they overlap nothing
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const int j0 = ((groups - 1) * D + d) * S;
                if (j0 * KS + kz >= nsteps) break;  // wave-uniform: chunks past the last step
                compute_chunk(a[d], xo[d], xo[(d + 1) % D][0], std::true_type{}, j0);
            }
        };
        switch (n_tiles) {
            case 1: reduce(std::integral_constant<int, 1>{}); break;
            case 2: reduce(std::integral_constant<int, 2>{}); break;
            case 3: reduce(std::integral_constant<int, 3>{}); break;
            default: reduce(std::integral_constant<int, 4>{}); break;
        }
    }

    // The partial sums of the reduction slices meet in LDS (the halo is no longer needed), added in
    // ascending slice order; the KS wavefronts of a channel group share the finishing of its R * NT
    // tiles, TPW each.
    float4_t fin[TPW];
    if (KS > 1) {
        float4_t *s_part = reinterpret_cast<float4_t *>(s_halo);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                s_part[(((kz * ncw + cw) * R + r) * NT + nt) * WAVE + lane] = acc[r][nt];
        __syncthreads();
#pragma unroll
        for (int q = 0; q < TPW; ++q) {
            const int t = kz * TPW + q;  // r * NT + nt
            fin[q] = s_part[((0 * ncw + cw) * R * NT + t) * WAVE + lane];
#pragma unroll
            for (int z = 1; z < KS; ++z) fin[q] += s_part[((z * ncw + cw) * R * NT + t) * WAVE + lane];
        }
    } else {
#pragma unroll
        for (int q = 0; q < TPW; ++q) fin[q] = acc[q / NT][q % NT];
    }
    // FIN: the sums go to LDS as pixel rows, behind the partial sums
    constexpr bool to_rows = FIN;
    unsigned char *s_rows = s_halo + (KS > 1 ? KS * ncw * R * NT * WAVE * 16 : 0);
    const int row_b = p.Co * (int)sizeof(E) + 16;
    if (FIN && KS == 1) __syncthreads();  // the halo is still being read by slower wavefronts
#pragma unroll
    for (int q = 0; q < TPW; ++q) {
        const int t = kz * TPW + q, nt = t % NT;
        const int ct = (cb * ncw + cw) * R + t / NT;
        if (ct >= co_tiles) continue;
        const int co = ct * 16 + kq * 4;  // lane holds channels co .. co + 3 of pixel (nt, l16)
        const int pix = nt * 16 + l16;
        if (pix >= n) continue;
        const int code = s_list[wv][pix], loc = code & 63;
        const size_t opix = ((size_t)b * p.Ho + out_y(loc >> 3)) * p.Wo + out_x(loc & 7);
        E *o = out + opix * p.Co + co;
        const bool vec = co + 3 < p.Co && (p.Co & 3) == 0;
        E4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = E(fin[q][i] + float(bv[q / NT][i]));
        if (ADD) {  // add_kernel's sequence on the rounded convolution result: s = a * wa; s = fma(b, wb, s)
            const bool upd = (code & 64) != 0, radd = (code & 128) != 0;
            const E wa = E(rs.wa), wb = E(rs.wb);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                E sum = E(0);
                if (radd) sum = rv[q][i] * wa;
                if (upd) sum = fma_t(v[i], wb, sum);
                v[i] = sum;
            }
        }
        if (to_rows) {  // (Co % 8 == 0: whole vectors)
            if (co < p.Co) *reinterpret_cast<E4 *>(s_rows + pix * row_b + co * (int)sizeof(E)) = v;
        } else if (vec) {
            *reinterpret_cast<E4 *>(o) = v;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (co + i < p.Co) o[i] = v[i];
        }
    }
    if (FIN) {
        __syncthreads();
        if (wv == 0 && inside && !any_px) out_mask[((size_t)b * p.Ho + oy) * p.Wo + ox] = 0;
#define DC_FIN_ACT(IT)                                                                                          \
    switch (fin_args.act) {                                                                                     \
        case DC_ACT_RELU: lds_finish<E, IT, DC_ACT_RELU>(fin_args, s_list[wv], n, tid, nthr, p.Co, out, out_mask, opix, s_rows, row_b, fq, ftr); break;   \
        case DC_ACT_RELU6: lds_finish<E, IT, DC_ACT_RELU6>(fin_args, s_list[wv], n, tid, nthr, p.Co, out, out_mask, opix, s_rows, row_b, fq, ftr); break; \
        case DC_ACT_LEAKY: lds_finish<E, IT, DC_ACT_LEAKY>(fin_args, s_list[wv], n, tid, nthr, p.Co, out, out_mask, opix, s_rows, row_b, fq, ftr); break; \
        default: lds_finish<E, IT, DC_ACT_LINEAR>(fin_args, s_list[wv], n, tid, nthr, p.Co, out, out_mask, opix, s_rows, row_b, fq, ftr); break;          \
    }
        if (fin_args.iters == 1) DC_FIN_ACT(1)
        else DC_FIN_ACT(2)
#undef DC_FIN_ACT
    }
}

// Small layers (few output tiles, as on the low-resolution branches of multi-branch networks):
// one 4x4 patch of output pixels x R channel tiles per workgroup, no compaction, no source
// table, no barrier before the reduction.  Lane (l16, kq) owns output pixel l16 of the patch; it
// requests the mask words of all its taps, and -- before they arrive -- the input and filter
// fragments of its first chunk of reduction steps, whose addresses depend on coordinates only.
// Fragments of taps that are out of bounds or inactive are zeroed by selection (every step is
// computed: at this size the instruction stream, not the MFMA count, is the kernel time);
// outputs are stored for updated pixels only.  KW wavefronts split the reduction steps round-robin.

// ADD: out = wa * residual [its mask] + wb * conv [updated pixels], out_mask = the union; with an
// activation the sum is accumulated in `prev` and its activated difference is emitted -- the
// arithmetic of add_kernel applied to the convolution result rounded to fp16, so the output
// equals that of the two separate launches bit for bit.
// MODE 2 (one wavefront holding every output channel of its 16 pixels: KW == 1, one channel
// block): the activation and truncation of DCActivation applied to the accumulators -- T = trunc
// + v, S = T + prev, D = act(S) - act(prev), one rounding each, the sequence of act_trunc_pixel;
// the keep statistics of a pixel are combined over its four k-quarter lanes.
template <typename E>
struct PatchEpi {
    E *prev, *trunc;
    float thr;
    int mode, act;
};

// LDS of a workgroup: s_red -- KW * R * WAVE partial sums (KW > 1), s_src -- KW tables of
// patch_tab_taps(taps) * 16 source indices.  (bx, by, bz): the workgroup's patch column, patch
// row and batch * channel block; kw: the wavefront's number among the KW of its workgroup.
__host__ __device__ constexpr int patch_tab_taps(int taps) { return taps + 12; }  // a pass writes up to 11 surplus taps

template <typename E, bool TR, int KW, int R, int S, int MODE, bool K3>
__device__ __forceinline__ void
conv_patch_body(const ConvP &p, const E *__restrict__ in, const E *__restrict__ wp,
                const E *__restrict__ bias, E *__restrict__ out,
                const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                int co_blocks, int ci_p, const PatchRes<E> &rs, const PatchEpi<E> &ep,
                int bx, int by, int bz, int kw, float4_t *s_red, int *s_src) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    constexpr bool ADD = MODE == 1, EPI = MODE == 2;
    static_assert(!EPI || KW == 1, "the fused activation needs all channels in one wavefront");
    constexpr int TAB_TAPS = patch_tab_taps(K3 ? 9 : MFMA_MAX_TAPS);
    const int b = bz / co_blocks, cb = bz % co_blocks;
    const int lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int oy = by * 4 + (l16 >> 2), ox = bx * 4 + (l16 & 3);
    const bool inside = oy < p.Ho && ox < p.Wo;
    const int K2 = K3 ? 9 : p.Kh * p.Kw;  // K3: a 3x3 kernel, tap arithmetic with constants
    const int Kw = K3 ? 3 : p.Kw;
    const int co_tiles = (p.Co + 15) >> 4;
    const int ksteps = ci_p >> 5;
    const int total = K2 * ksteps;
    const E *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    const E *wfrag[R];
#pragma unroll
    for (int r = 0; r < R; ++r)  // surplus channel tiles re-read the last one and are not stored
        wfrag[r] = wp + (size_t)min(cb * R + r, co_tiles - 1) * total * 512 + lane * 8;

    // Source table of this wavefront in LDS: s_src[tap * 16 + pixel] = input pixel index read by
    // the lane's output pixel through `tap`, or -1 if it is out of bounds.  The four k-quarter
    // lanes of a pixel share the taps (kq, kq + 4, ...), each also fetches the mask word of its
    // taps; the activity bits are then combined across the four lanes.
    int *src_tab = s_src + kw * (TAB_TAPS * 16);
    unsigned long long bits = 0;
    for (int t0 = 0; t0 < K2; t0 += 12) {
        int word[3], src[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            // straight-line (selects instead of branches): the three mask words of a lane are
            // requested back to back; the table has room for the surplus taps of the last pass
            const int tap = t0 + kq + 4 * j;
            const int tc = min(tap, K2 - 1);
            const int ky = tc / Kw, kx = tc - ky * Kw;
            int iy = 0, ix = 0;
            const bool oky = tap_src<TR>(oy, ky, p.sh, p.dh, p.pt, p.Hi, iy);
            const bool okx = tap_src<TR>(ox, kx, p.sw, p.dw, p.pl, p.Wi, ix);
            src[j] = (tap < K2 && inside && oky && okx) ? iy * p.Wi + ix : -1;
            src_tab[tap * 16 + l16] = src[j];
            word[j] = mb[max(src[j], 0)];
        }
#pragma unroll
        for (int j = 0; j < 3; ++j)
            if (src[j] >= 0 && word[j] != 0) bits |= 1ull << (t0 + kq + 4 * j);
    }
    const size_t opix = ((size_t)b * p.Ho + min(oy, p.Ho - 1)) * p.Wo + min(ox, p.Wo - 1);
    int rword = 0;
    if (ADD) rword = rs.mask[opix];
    // Steps of this wavefront: s = kw, kw + KW, ...; (tap, channel step) advance with it and are
    // wave-uniform, so they live in scalar registers.
    int n_tap = 0, n_ks = kw;
    while (n_ks >= ksteps) { n_ks -= ksteps; ++n_tap; }
    auto load_chunk = [&](E8 (&a)[S][R], E8 (&x)[S], int (&tp)[S]) {
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int tap = min(n_tap, K2 - 1), ks = n_tap < K2 ? n_ks : ksteps - 1;  // past the end: last step again
            tp[i] = tap;
            const int k = min((ks << 5) + kq * 8, p.Ci - 8);
            const int sp = src_tab[tap * 16 + l16];
#pragma unroll
            for (int r = 0; r < R; ++r)
                a[i][r] = *reinterpret_cast<const E8 *>(wfrag[r] + (size_t)(tap * ksteps + ks) * 512);
            x[i] = *reinterpret_cast<const E8 *>(inb + (size_t)max(sp, 0) * p.Ci + k);
            n_ks += KW;
            while (n_ks >= ksteps) { n_ks -= ksteps; ++n_tap; }
        }
    };

    // eager: the first chunk of fragments is requested while the mask words are in flight
    E8 a[S][R], x[S];
    int tp[S];
    load_chunk(a, x, tp);
    bits |= __shfl_xor(bits, 16, WAVE);
    bits |= __shfl_xor(bits, 32, WAVE);
    const bool upd = bits != 0;
    const bool radd = ADD && inside && rword != 0;
    // with the fused activation the mask word of an updated pixel is its keep decision, below
    if (cb == 0 && kw == 0 && kq == 0 && inside && !(EPI && upd)) out_mask[opix] = (upd || radd) ? 1 : 0;
    const bool reduce = ballot(upd) != 0;  // the same in every wavefront of the workgroup
    if (!reduce && ballot(radd) == 0) return;
    E4 eq[R], etr[R];  // cached state of the fused activation, requested before the reduction
    if (EPI) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const size_t off = (upd ? opix : 0) * p.Co + min((cb * R + r) * 16 + kq * 4, p.Co - 4);
            eq[r] = *reinterpret_cast<const E4 *>(ep.prev + off);
            etr[r] = *reinterpret_cast<const E4 *>(ep.trunc + off);
        }
    }
    // operands of the fused sum, requested now so that they arrive during the reduction
    E4 rv[R], qv[R];
    if (ADD) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int co = min((cb * R + r) * 16 + kq * 4, ((p.Co + 3) & ~3) - 4);
            if ((p.Co & 3) == 0) {
                rv[r] = *reinterpret_cast<const E4 *>(rs.values + opix * p.Co + co);
                if (rs.act > 0) qv[r] = *reinterpret_cast<const E4 *>(rs.prev + opix * p.Co + co);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int c = min((cb * R + r) * 16 + kq * 4 + i, p.Co - 1);
                    rv[r][i] = rs.values[opix * p.Co + c];
                    if (rs.act > 0) qv[r][i] = rs.prev[opix * p.Co + c];
                }
            }
        }
    }

    float4_t acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s0 = kw; s0 < total && reduce; s0 += S * KW) {
        if (s0 != kw) load_chunk(a, x, tp);
#pragma unroll
        for (int i = 0; i < S; ++i) {
            // straight-line: a step past the end or an invalid (tap, pixel) pair multiplies zeros
            const E8 xz = keep8(x[i], s0 + i * KW < total && ((bits >> tp[i]) & 1ull));
#pragma unroll
            for (int r = 0; r < R; ++r)
                acc[r] = Elem16<E>::mfma(a[i][r], xz, acc[r]);
        }
    }
    if (KW > 1 && reduce) {
#pragma unroll
        for (int r = 0; r < R; ++r) s_red[(kw * R + r) * WAVE + lane] = acc[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if ((r % KW) != kw) continue;  // wavefront kw finishes channel tiles kw, kw + KW, ...
            float4_t sum = s_red[r * WAVE + lane];
#pragma unroll
            for (int q = 1; q < KW; ++q) sum += s_red[(q * R + r) * WAVE + lane];
            acc[r] = sum;
        }
    }
    if (EPI) {
        const E thr = E(ep.thr);
        auto finish = [&](auto act_c) {  // the activation as a compile-time constant
            constexpr int ACTC = decltype(act_c)::value;
            E4 t[R], sm[R], d[R];
            bool hit = false;
            float sq = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int co = (cb * R + r) * 16 + kq * 4;
                const bool live = upd && cb * R + r < co_tiles && co < p.Co;
                E4 bh = zero4<E>();
                if (bias != nullptr) bh = *reinterpret_cast<const E4 *>(bias + min(co, p.Co - 4));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const E v = E(acc[r][i] + float(bh[i]));
                    t[r][i] = etr[r][i] + v;
                    sm[r][i] = t[r][i] + eq[r][i];
                    d[r][i] = act_apply<E>(sm[r][i], ACTC) - act_apply<E>(eq[r][i], ACTC);
                    if (live) {
                        hit |= tabs(d[r][i]) > thr;
                        sq += float(d[r][i]) * float(d[r][i]);
                    }
                }
            }
            bool keep;
            if (ep.mode == DC_TRUNC_MAX) {
                const uint64_t bl = ballot(hit);
                keep = ((bl >> l16) & 0x0001000100010001ull) != 0;
            } else {
                sq += __shfl_xor(sq, 16, WAVE);
                sq += __shfl_xor(sq, 32, WAVE);
                if (ep.mode == DC_TRUNC_RMS) sq /= float(p.Co);
                keep = sqrtf(sq) > float(thr);
            }
            if (!upd) return;
            if (kq == 0) out_mask[opix] = keep ? 1 : 0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int co = (cb * R + r) * 16 + kq * 4;
                if (cb * R + r >= co_tiles || co >= p.Co) continue;
                const size_t off = opix * p.Co + co;
                if (keep) {
                    *reinterpret_cast<E4 *>(ep.prev + off) = sm[r];
                    *reinterpret_cast<E4 *>(out + off) = d[r];
                    if (bits_set8(etr[r])) *reinterpret_cast<E4 *>(ep.trunc + off) = zero4<E>();  // else zero already
                } else {
                    *reinterpret_cast<E4 *>(ep.trunc + off) = t[r];
                }
            }
        };
        switch (ep.act) {
            case DC_ACT_RELU: finish(std::integral_constant<int, DC_ACT_RELU>{}); break;
            case DC_ACT_RELU6: finish(std::integral_constant<int, DC_ACT_RELU6>{}); break;
            case DC_ACT_LEAKY: finish(std::integral_constant<int, DC_ACT_LEAKY>{}); break;
            case DC_ACT_SIGMOID: finish(std::integral_constant<int, DC_ACT_SIGMOID>{}); break;
            case DC_ACT_SWISH: finish(std::integral_constant<int, DC_ACT_SWISH>{}); break;
            default: finish(std::integral_constant<int, DC_ACT_LINEAR>{}); break;
        }
        return;
    }
    if (!(upd || radd)) return;
    E *o = out + opix * p.Co;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (KW > 1 && (r % KW) != kw) continue;
        const int ct = cb * R + r, co = ct * 16 + kq * 4;
        if (ct >= co_tiles) continue;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias != nullptr) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (co + i < p.Co) bv[i] = float(bias[co + i]);
        }
        E4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = E(acc[r][i] + bv[i]);
        E4 q;
        if (ADD) {  // add_kernel's sequence: s = a * wa; s = fma(b, wb, s); n = s + prev; ...
            const E wa = E(rs.wa), wb = E(rs.wb);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                E sum = E(0);
                if (radd) sum = rv[r][i] * wa;
                if (upd) sum = fma_t(v[i], wb, sum);
                if (rs.act > 0) {
                    const E n = sum + qv[r][i];
                    sum = act_apply<E>(n, rs.act) - act_apply<E>(qv[r][i], rs.act);
                    q[i] = n;
                }
                v[i] = sum;
            }
        }
        if (co + 3 < p.Co && (p.Co & 3) == 0) {
            *reinterpret_cast<E4 *>(o + co) = v;
            if (ADD && rs.act > 0) *reinterpret_cast<E4 *>(rs.prev + opix * p.Co + co) = q;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (co + i < p.Co) {
                    o[co + i] = v[i];
                    if (ADD && rs.act > 0) rs.prev[opix * p.Co + co + i] = q[i];
                }
        }
    }
}

template <typename E, bool TR, int KW, int R, int S, int MODE, bool K3>
__global__ void __launch_bounds__(KW * WAVE)
conv_patch_mfma_kernel(ConvP p, const E *__restrict__ in, const E *__restrict__ wp,
                       const E *__restrict__ bias, E *__restrict__ out,
                       const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask,
                       int co_blocks, int ci_p, PatchRes<E> rs, PatchEpi<E> ep) {
    __shared__ float4_t s_red[KW > 1 ? KW * R * WAVE : 1];
    __shared__ int s_src[KW * patch_tab_taps(K3 ? 9 : MFMA_MAX_TAPS) * 16];
    conv_patch_body<E, TR, KW, R, S, MODE, K3>(p, in, wp, bias, out, mask, out_mask, co_blocks, ci_p, rs, ep,
                                               blockIdx.x, blockIdx.y, blockIdx.z, wave_id(), s_red, s_src);
}

// Several independent small layers -- the parallel branches of a multi-resolution network -- in
// ONE launch: every workgroup looks up the layer its number falls into and runs that layer's
// arrangement of conv_patch_mfma_kernel unchanged (same code, same summation order: results are
// those of the separate launches bit for bit).  Workgroups have as many wavefronts as the
// longest reduction of the group splits over; the surplus wavefronts of the other layers leave
// at once.  3 x 3 kernels only (the source tables of all arrangements share one LDS block).
constexpr int GROUP_MAX = CONV_GROUP_MAX;

template <typename E>
struct PatchItem {
    ConvP p;
    const E *in, *wp, *bias;
    E *out;
    const int32_t *mask;
    int32_t *out_mask;
    int co_blocks, ci_p;
    PatchRes<E> rs;
    PatchEpi<E> ep;
    int kwv, rv, mode;  // arrangement: reduction slices, channel tiles per wavefront, 0 plain / 1 sum / 2 activation
    int gx, gy;         // patch columns and rows
    int first;          // number of this layer's first workgroup
};

template <typename E>
struct PatchGroup {
    int n;
    PatchItem<E> it[GROUP_MAX];
};

template <typename E>
__global__ void __launch_bounds__(8 * WAVE)
conv_patch_group_kernel(PatchGroup<E> g) {
    __shared__ float4_t s_red[8 * 2 * WAVE];
    __shared__ int s_src[8 * patch_tab_taps(9) * 16];
    int idx = 0;
#pragma unroll
    for (int i = 1; i < GROUP_MAX; ++i)
        if (i < g.n && (int)blockIdx.x >= g.it[i].first) idx = i;
    const PatchItem<E> &it = g.it[idx];
    if (wave_id() >= it.kwv) return;  // wave-uniform; the barrier counts the remaining wavefronts
    const int local = blockIdx.x - it.first;
    const int bx = local % it.gx, by = (local / it.gx) % it.gy, bz = local / (it.gx * it.gy);
#define DC_GROUP_BODY(KWV, RV, SV, MV)                                                                               \
    conv_patch_body<E, false, KWV, RV, SV, MV, true>(it.p, it.in, it.wp, it.bias, it.out, it.mask, it.out_mask,     \
                                                     it.co_blocks, it.ci_p, it.rs, it.ep, bx, by, bz, wave_id(), s_red, s_src)
#define DC_GROUP_MODE(KWV, RV, SV)                         \
    do {                                                   \
        if (it.mode == 1) DC_GROUP_BODY(KWV, RV, SV, 1);   \
        else DC_GROUP_BODY(KWV, RV, SV, 0);                \
    } while (0)
    if (it.kwv == 1) {
        if (it.mode == 2) { if (it.rv == 2) DC_GROUP_BODY(1, 2, 9, 2); else DC_GROUP_BODY(1, 1, 9, 2); }
        else if (it.rv == 2) DC_GROUP_MODE(1, 2, 9);
        else DC_GROUP_MODE(1, 1, 9);
    } else if (it.kwv == 4) {
        if (it.rv == 2) DC_GROUP_MODE(4, 2, 5); else DC_GROUP_MODE(4, 1, 9);
    } else {
        if (it.rv == 2) DC_GROUP_MODE(8, 2, 6); else DC_GROUP_MODE(8, 1, 9);
    }
#undef DC_GROUP_MODE
#undef DC_GROUP_BODY
}

// One-time relayout of a reference-layout fp16 filter [Cin pad 2][K][K][Cout pad 2] (channel
// pairs swizzled: W[ci][co] is stored at row ci ^ (co & 1); swz == 0: the plain [Cin][K][K][Cout]
// layout of bfloat16 filters) into MFMA fragment order
// [Cout tile of 16][tap][Cin step of 32][lane 0..63][8]: lane (kq * 16 + r) of a fragment holds
// input channels kq * 8 .. + 8 of output channel r, so one A operand of
// v_mfma_f32_16x16x32_f16 is a single contiguous 1 KB read (16 bytes per lane, consecutive
// lanes at consecutive addresses).  Channels past Cin / Cout are zero.
__global__ void pack_filter_kernel(const uint16_t *__restrict__ f, uint16_t *__restrict__ wp, int Ci,
                                   int Co, int K2, int w_co, int ci_p, int co_p, int swz) {
    const size_t total = (size_t)co_p * K2 * ci_p;
    const int ksteps = ci_p >> 5;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const int e = int(i & 7), lane = int((i >> 3) & 63);
        const size_t frag = i >> 9;
        const int step = int(frag % ksteps);
        const int tap = int((frag / ksteps) % K2);
        const int ct = int(frag / ((size_t)ksteps * K2));
        const int co = ct * 16 + (lane & 15);
        const int ci = step * 32 + (lane >> 4) * 8 + e;
        uint16_t v = 0;  // 16-bit elements of either type are moved as they are
        if (ci < Ci && co < Co) v = f[((size_t)(ci ^ (swz ? (co & 1) : 0)) * K2 + tap) * w_co + co];
        wp[i] = v;
    }
}


// ------------------------------------------------------- few input channels on the matrix cores
// Stems of large frames (Cin <= 4, window up to 8 x 8, stride <= 2, Cout <= 64, fp16).  With the
// input channels padded to 4 in LDS, the 32 reduction elements of one MFMA step are one window
// ROW: k = kx * 4 + ci for kx = 0..7, so the input fragment of lane (pixel, kq) -- elements
// kq * 8 .. kq * 8 + 7 -- is simply the two neighbouring halo pixels kx = 2 kq, 2 kq + 1 of that
// row, 16 contiguous bytes; no im2col copy exists.  Window columns past Kw and channel 3 of an
// RGB input meet zero weights in the packed filter ([Cout tile][ky][lane][8], see
// pack_stem_filter_kernel); inactive and out-of-bounds pixels are staged as zeros.
// Workgroup = 8 x 8 output pixels, wavefront w = rows 2w, 2w + 1 x all R channel tiles, so the
// keep decision of the fused activation stays inside the wavefront.  The halo's update mask is
// kept as one bit row per halo row; an output is updated if its window meets a set bit.
constexpr int STEM_K = 8;
template <typename E, int R, int ACT>
__global__ void __launch_bounds__(256)
conv_stem_mfma_kernel(ConvP p, const E *__restrict__ in, const E *__restrict__ wp,
                      const E *__restrict__ bias, E *__restrict__ out,
                      const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, EpiP epi,
                      int hal_h, int hal_wp, int lazy) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    extern __shared__ __align__(16) unsigned char s_mem[];
    E *s_x = reinterpret_cast<E *>(s_mem);                       // [hal_h][hal_wp][4]
    unsigned *s_row = reinterpret_cast<unsigned *>(s_x + hal_h * hal_wp * 4);  // [hal_h]
    const int b = blockIdx.z, ty0 = blockIdx.y * TILE, tx0 = blockIdx.x * TILE;
    const int tid = threadIdx.x, wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int iy0 = ty0 * p.sh - p.pt, ix0 = tx0 * p.sw - p.pl;
    // filter fragments of the wavefront's R channel tiles: requested first, used last (surplus
    // tiles re-read the last one and are not stored)
    const int co_tiles = (p.Co + 15) >> 4;
    E8 a[R][STEM_K];
    auto load_filter = [&]() {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int ky = 0; ky < STEM_K; ++ky)
                a[r][ky] = *reinterpret_cast<const E8 *>(wp + ((size_t)(min(r, co_tiles - 1) * p.Kh + min(ky, p.Kh - 1)) * WAVE + lane) * 8);
    };
    if (!lazy) load_filter();  // lazy: a tile without an update does not fetch its 16 KB per wavefront
    E4 bv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        bv[r] = zero4<E>();
        if (bias != nullptr) bv[r] = *reinterpret_cast<const E4 *>(bias + min(r * 16 + kq * 4, p.Co - 4));
    }
    if (tid < hal_h) s_row[tid] = 0;
    __syncthreads();
    const E *inb = in + (size_t)b * p.Hi * p.Wi * p.Ci;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    for (int hp = tid; hp < hal_h * hal_wp; hp += 256) {
        const int hy = hp / hal_wp, hx = hp - hy * hal_wp;
        const int iy = iy0 + hy, ix = ix0 + hx;
        const bool ok = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
        const size_t pix = ok ? (size_t)iy * p.Wi + ix : 0;
        const int word = mb[pix];
        E4 v = zero4<E>();
        // small maps: the pixel is requested together with its mask word (one round trip);
        // lazy (large maps, where instructions and bytes count, not the latency chain): only
        // updated pixels are read at all
        if (!lazy || (ok && word != 0)) {
#pragma unroll
            for (int ci = 0; ci < 4; ++ci) v[ci] = inb[pix * p.Ci + min(ci, p.Ci - 1)];
        }
        const bool m = ok && word != 0;
#pragma unroll
        for (int ci = 0; ci < 4; ++ci) v[ci] = (m && ci < p.Ci) ? v[ci] : E(0);
        *reinterpret_cast<E4 *>(s_x + hp * 4) = v;
        if (m) atomicOr(&s_row[hy], 1u << hx);
    }
    __syncthreads();

    const int ly = wave * 2 + (l16 >> 3), lx = l16 & 7;
    const int oy = ty0 + ly, ox = tx0 + lx;
    const bool inside = oy < p.Ho && ox < p.Wo;
    unsigned any = 0;
    for (int ky = 0; ky < p.Kh; ++ky) any |= (s_row[ly * p.sh + ky] >> (lx * p.sw)) & ((1u << p.Kw) - 1u);
    const bool upd = inside && any != 0;
    const size_t po = ((size_t)b * p.Ho + oy) * p.Wo + ox;
    if (inside && kq == 0 && (ACT < 0 || !upd)) out_mask[po] = upd ? 1 : 0;
    if (ballot(upd) == 0) return;
    if (lazy) load_filter();

    // cached state of the fused epilogue, requested before the contraction
    E4 q[R], tr[R];
    if (ACT >= 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const size_t off = (upd ? po : 0) * p.Co + min(r * 16 + kq * 4, p.Co - 4);
            q[r] = *reinterpret_cast<const E4 *>((const E *)epi.prev + off);
            tr[r] = *reinterpret_cast<const E4 *>((const E *)epi.trunc + off);
        }
    }
    float4_t acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ky = 0; ky < STEM_K; ++ky) {
        if (ky < p.Kh) {  // uniform
            const E *xp = s_x + ((ly * p.sh + ky) * hal_wp + lx * p.sw + 2 * kq) * 4;
            const E4 x0 = *reinterpret_cast<const E4 *>(xp), x1 = *reinterpret_cast<const E4 *>(xp + 4);
            const E8 x = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = Elem16<E>::mfma(a[r][ky], x, acc[r]);
        }
    }
    E4 v[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) v[r][i] = E(acc[r][i] + float(bv[r][i]));
    if (ACT < 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int co = r * 16 + kq * 4;
            if (upd && co < p.Co) *reinterpret_cast<E4 *>(out + po * p.Co + co) = v[r];
        }
        return;
    }
    // activation + truncation, the operations and roundings of act_trunc_pixel; the statistics
    // of a pixel are combined over its four kq lanes
    constexpr int ACTC = ACT < 0 ? 0 : ACT;
    const E thr = E(epi.thr);
    E4 t[R], sm[R], d[R];
    bool hit = false;
    float sq = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const bool live = upd && r * 16 + kq * 4 < p.Co;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            t[r][i] = tr[r][i] + v[r][i];
            sm[r][i] = t[r][i] + q[r][i];
            d[r][i] = act_apply<E>(sm[r][i], ACTC) - act_apply<E>(q[r][i], ACTC);
            if (live) {
                hit |= tabs(d[r][i]) > thr;
                sq += float(d[r][i]) * float(d[r][i]);
            }
        }
    }
    bool keep;
    if (epi.mode == DC_TRUNC_MAX) {
        const uint64_t bl = ballot(hit);
        keep = ((bl >> l16) & 0x0001000100010001ull) != 0;
    } else {
        sq += __shfl_xor(sq, 16, WAVE);
        sq += __shfl_xor(sq, 32, WAVE);
        if (epi.mode == DC_TRUNC_RMS) sq /= float(p.Co);
        keep = sqrtf(sq) > float(thr);
    }
    if (!upd) return;
    if (kq == 0) out_mask[po] = keep ? 1 : 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int co = r * 16 + kq * 4;
        if (co >= p.Co) continue;
        const size_t off = po * p.Co + co;
        if (keep) {
            *reinterpret_cast<E4 *>((E *)epi.prev + off) = sm[r];
            *reinterpret_cast<E4 *>(out + off) = d[r];
            if (bits_set8(tr[r])) *reinterpret_cast<E4 *>((E *)epi.trunc + off) = zero4<E>();  // else zero already
        } else {
            *reinterpret_cast<E4 *>((E *)epi.trunc + off) = t[r];
        }
    }
}

// ------------------------------------------------------- thin layers on the matrix cores
// K x K convolutions (window up to 3 x 3, stride <= 2) with 8 or 16 input channels and up to 64
// output channels on large maps, where the LDS-halo kernel spends a whole reduction step of 32 on
// every tap and stores in 8-byte pieces.  Here a reduction step holds 32 / CIN TAPS: lane
// (pixel, kq) of the input fragment reads the 16 bytes of tap s * TPS + kq * 8 / CIN, channels
// (kq * 8) % CIN .. + 7, straight from the staged halo -- 5 steps instead of 9 for 16 channels,
// 3 for 8 -- and the filter fragments (gathered once per wavefront from the packed filter, whose
// fragment (channel tile, tap) holds the same 16 bytes in lane (ci / 8) * 16 + co) stay in registers.
// Workgroup = 8 x 8 output pixels, wavefront w = rows 2w, 2w + 1 x all R channel tiles.  The
// rounded result goes through a wavefront-private LDS tile into pixel rows; output and, MODE 2,
// the activation / maximum-norm truncation of the layer work on rows in 16-byte pieces (the
// operations and roundings of act_trunc_pixel; the keep decision of a pixel through an LDS flag),
// the cached state requested before the contraction.  lazy (maps of 2^18 pixels and more): only
// updated pixels are read at all.  MODE 0: convolution only.
template <typename E, int CIN, int R, int MODE, int ACT>
__global__ void __launch_bounds__(256)
conv_thin_mfma_kernel(ConvP p, const E *__restrict__ in, const E *__restrict__ wp,
                      const E *__restrict__ bias, E *__restrict__ out,
                      const int32_t *__restrict__ mask, int32_t *__restrict__ out_mask, EpiP epi,
                      int hal_h, int hal_w, int lazy) {
    typedef typename Elem16<E>::v4 E4;
    typedef typename Elem16<E>::v8 E8;
    static_assert(CIN == 8 || CIN == 16, "8 or 16 input channels");
    constexpr int TPS = 32 / CIN;            // taps per reduction step
    constexpr int NS = (9 + TPS - 1) / TPS;  // reduction steps of a window of up to nine taps
    constexpr int CV = CIN / 8;              // 16-byte pieces per staged pixel
    constexpr int ROWB = R * 32 + 16;        // bytes of a staged output row: padded, rows start in different banks
    constexpr int PIECES = (16 * R * 2 + WAVE - 1) / WAVE;
    extern __shared__ __align__(16) unsigned char s_mem[];
    E *s_x = reinterpret_cast<E *>(s_mem);                                     // [hal_h * hal_w][CIN]
    unsigned char *s_v = s_mem + hal_h * hal_w * CIN * 2 + wave_id() * 16 * ROWB;  // [4 wavefronts][16][ROWB]
    unsigned *s_row = reinterpret_cast<unsigned *>(s_mem + hal_h * hal_w * CIN * 2 + 4 * 16 * ROWB);  // [hal_h]
    __shared__ int s_keep[4][16];
    const int b = blockIdx.z, ty0 = blockIdx.y * TILE, tx0 = blockIdx.x * TILE;
    const int tid = threadIdx.x, wave = wave_id(), lane = lane_id();
    const int l16 = lane & 15, kq = lane >> 4;
    const int iy0 = ty0 * p.sh - p.pt, ix0 = tx0 * p.sw - p.pl;
    const int K2 = p.Kh * p.Kw;
    const int co_tiles = (p.Co + 15) >> 4;
    const int rc = p.Co >> 3;  // 16-byte pieces of an output row (Cout % 8 == 0)
    // this lane's tap and 8-channel piece in reduction step st
    const int tsub = CIN == 16 ? kq >> 1 : kq, c8 = CIN == 16 ? kq & 1 : 0;
    E8 a[R][NS];
    auto load_filter = [&]() {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int st = 0; st < NS; ++st) {
                const int t = st * TPS + tsub;
                const E8 w = *reinterpret_cast<const E8 *>(
                    wp + ((size_t)(min(r, co_tiles - 1) * K2 + min(t, K2 - 1)) * WAVE + c8 * 16 + l16) * 8);
                a[r][st] = keep8(w, t < K2);  // taps past the window meet zero weights
            }
    };
    if (!lazy) load_filter();  // lazy: a tile without an update does not fetch the filter
    E4 bv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        bv[r] = zero4<E>();
        if (bias != nullptr) bv[r] = *reinterpret_cast<const E4 *>(bias + min(r * 16 + kq * 4, p.Co - 4));
    }
    if (tid < hal_h) s_row[tid] = 0;
    __syncthreads();
    const E *inb = in + (size_t)b * p.Hi * p.Wi * CIN;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    for (int hp = tid; hp < hal_h * hal_w; hp += 256) {
        const int hy = hp / hal_w, hx = hp - hy * hal_w;
        const int iy = iy0 + hy, ix = ix0 + hx;
        const bool ok = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
        const size_t pix = ok ? (size_t)iy * p.Wi + ix : 0;
        const int word = mb[pix];
        const bool m = ok && word != 0;
        E8 v[CV] = {};
        // small maps: the pixel is requested together with its mask word (one round trip);
        // lazy: only updated pixels are read
        if (!lazy || m) {
#pragma unroll
            for (int c = 0; c < CV; ++c) v[c] = *reinterpret_cast<const E8 *>(inb + pix * CIN + c * 8);
        }
#pragma unroll
        for (int c = 0; c < CV; ++c) *reinterpret_cast<E8 *>(s_x + hp * CIN + c * 8) = keep8(v[c], m);
        if (m) atomicOr(&s_row[hy], 1u << hx);
    }
    __syncthreads();

    const int ly = wave * 2 + (l16 >> 3), lx = l16 & 7;
    const int oy = ty0 + ly, ox = tx0 + lx;
    const bool inside = oy < p.Ho && ox < p.Wo;
    unsigned any = 0;
    for (int ky = 0; ky < p.Kh; ++ky) any |= (s_row[ly * p.sh + ky] >> (lx * p.sw)) & ((1u << p.Kw) - 1u);
    const bool upd = inside && any != 0;
    const size_t po = ((size_t)b * p.Ho + oy) * p.Wo + ox;
    if (inside && kq == 0 && (MODE == 0 || !upd)) out_mask[po] = upd ? 1 : 0;
    const uint64_t bu = ballot(upd);
    if (bu == 0) return;
    if (lazy) load_filter();

    // the row pieces this lane finishes: piece c = lane + i * 64 of the wavefront's 16 rows is piece
    // c % rc of pixel c / rc; the cached state is requested now, before the contraction
    int ppix[PIECES], pcol[PIECES];
    bool pon[PIECES];
    size_t poff[PIECES], ppo[PIECES];
    E8 qrow[MODE == 2 ? PIECES : 1], trow[MODE == 2 ? PIECES : 1];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int c = lane + i * WAVE;
        const int r = min(c / rc, 15), cc = c - (c / rc) * rc;
        ppix[i] = r;
        pcol[i] = cc * 8;
        pon[i] = c < 16 * rc && ((bu >> r) & 1);
        const int ry = ty0 + wave * 2 + (r >> 3), rx = tx0 + (r & 7);
        ppo[i] = pon[i] ? ((size_t)b * p.Ho + ry) * p.Wo + rx : 0;
        poff[i] = ppo[i] * p.Co + (pon[i] ? pcol[i] : 0);
        if (MODE == 2) {
            qrow[i] = *reinterpret_cast<const E8 *>((const E *)epi.prev + poff[i]);
            trow[i] = *reinterpret_cast<const E8 *>((const E *)epi.trunc + poff[i]);
        }
    }
    float4_t acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < NS; ++st) {
        if (st * TPS < K2) {  // uniform
            const int t = min(st * TPS + tsub, K2 - 1);
            const int ky = t / p.Kw, kx = t - ky * p.Kw;
            const E8 x = *reinterpret_cast<const E8 *>(s_x + ((ly * p.sh + ky) * hal_w + lx * p.sw + kx) * CIN + c8 * 8);
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = Elem16<E>::mfma(a[r][st], x, acc[r]);
        }
    }
    // rounded result into the wavefront's LDS tile, pixel rows contiguous
#pragma unroll
    for (int r = 0; r < R; ++r) {
        E4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = E(acc[r][i] + float(bv[r][i]));
        *reinterpret_cast<E4 *>(s_v + l16 * ROWB + r * 32 + kq * 8) = v;
    }
    if (MODE == 2 && lane < 16) s_keep[wave][lane] = 0;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    E8 vrow[PIECES];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) vrow[i] = *reinterpret_cast<const E8 *>(s_v + ppix[i] * ROWB + pcol[i] * 2);
    if (MODE == 0) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
            if (pon[i]) *reinterpret_cast<E8 *>(out + poff[i]) = vrow[i];
        return;
    }
    constexpr int ACTC = ACT < 0 ? 0 : ACT;
    const E thr = E(epi.thr);
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        bool hit = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const E t = trow[i][j] + vrow[i][j];
            const E sm = t + qrow[i][j];
            const E d = act_apply<E>(sm, ACTC) - act_apply<E>(qrow[i][j], ACTC);
            hit |= tabs(d) > thr;
        }
        if (pon[i] && hit) s_keep[wave][ppix[i]] = 1;
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // second pass: T, S, D again (a handful of operations, cheaper than holding them)
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        if (!pon[i]) continue;
        const bool keep = s_keep[wave][ppix[i]] != 0;
        if (pcol[i] == 0) out_mask[ppo[i]] = keep ? 1 : 0;
        E8 tv, sv, dv, z;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            tv[j] = trow[i][j] + vrow[i][j];
            sv[j] = tv[j] + qrow[i][j];
            dv[j] = act_apply<E>(sv[j], ACTC) - act_apply<E>(qrow[i][j], ACTC);
            z[j] = E(0);
        }
        if (keep) {
            *reinterpret_cast<E8 *>((E *)epi.prev + poff[i]) = sv;
            *reinterpret_cast<E8 *>(out + poff[i]) = dv;
            if (bits_set16(trow[i])) *reinterpret_cast<E8 *>((E *)epi.trunc + poff[i]) = z;  // else zero already
        } else {
            *reinterpret_cast<E8 *>((E *)epi.trunc + poff[i]) = tv;
        }
    }
}

// Filter of conv_stem_mfma_kernel: fragment (channel tile, ky) holds, for lane (l16, kq) and
// element e, W[co = tile * 16 + l16][ky][kx = (kq * 8 + e) / 4][ci = (kq * 8 + e) % 4], zero past
// Kw, Cin and Cout.  Reads the processed fp16 layout (rows swizzled by the output parity) or,
// swz == 0, the plain layout of bfloat16 filters; 16-bit elements of either type move as they are.
__global__ void pack_stem_filter_kernel(const uint16_t *__restrict__ f, uint16_t *__restrict__ wp, int Ci,
                                        int Co, int Kh, int Kw, int w_co, int co_tiles, int swz) {
    const int total = co_tiles * Kh * 512;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const int e = i & 7, lane = (i >> 3) & 63, frag = i >> 9;
        const int ky = frag % Kh, ct = frag / Kh;
        const int co = ct * 16 + (lane & 15), k = (lane >> 4) * 8 + e;
        const int kx = k >> 2, ci = k & 3;
        uint16_t v = 0;
        if (kx < Kw && ci < Ci && co < Co) v = f[((size_t)(ci ^ (swz ? (co & 1) : 0)) * Kh * Kw + ky * Kw + kx) * w_co + co];
        wp[i] = v;
    }
}

inline bool stem_eligible(const dc_geometry &g, int dtype) {
    return (dtype == DC_F16 || dtype == DC_BF16) && g.groups == 1 && g.in_c <= 4 && g.kernel_h <= STEM_K && g.kernel_w <= STEM_K &&
           g.dilation_h == 1 && g.dilation_w == 1 && g.stride_h <= 2 && g.stride_w <= 2 && g.out_c % 4 == 0 &&
           g.out_c <= 64;
}

inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

// Raises a kernel's dynamic LDS limit to 112 KB, once per kernel and device (the attribute belongs
// to the device's copy of the function); a plain host call, nothing is put on a stream.
template <typename K>
hipError_t allow_large_lds(K *kernel) {
    static std::atomic<uint64_t> done{0};  // one bit per device; devices past 63 ask every time
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 64 && ((done.load(std::memory_order_relaxed) >> dev) & 1ull)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 112 << 10);
    if (e == hipSuccess && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
    return e;
}

inline bool mfma_eligible(const dc_geometry &g, int dtype) {
    return (dtype == DC_F16 || dtype == DC_BF16) && g.groups == 1 && g.in_c % 8 == 0 && g.in_c >= 8;
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
    if (!transposed && stem_eligible(g, dtype)) return (int64_t)ceil_div(g.out_c, 16) * g.kernel_h * 1024;
    if (!mfma_eligible(g, dtype)) return 0;
    return (int64_t)round_up(g.out_c, 16) * g.kernel_h * g.kernel_w * round_up(g.in_c, 32) * 2;
}

hipError_t launch_pack_filter(const dc_geometry &g, const void *filter, void *packed, int dtype,
                              bool transposed, hipStream_t s) {
    if (!transposed && stem_eligible(g, dtype)) {
        note_kernel("pack_stem_filter_kernel");
        const int co_tiles = ceil_div(g.out_c, 16);
        pack_stem_filter_kernel<<<ceil_div(co_tiles * g.kernel_h * 512, 256), 256, 0, s>>>(
            (const uint16_t *)filter, (uint16_t *)packed, g.in_c, g.out_c, g.kernel_h, g.kernel_w,
            dtype == DC_F16 ? g.out_c + (g.out_c & 1) : g.out_c, co_tiles, dtype == DC_F16 ? 1 : 0);
        return hipGetLastError();
    }
    if (!mfma_eligible(g, dtype)) return hipSuccess;
    const int K2 = g.kernel_h * g.kernel_w;
    const int ci_p = round_up(g.in_c, 32), co_p = round_up(g.out_c, 16);
    const size_t total = (size_t)co_p * K2 * ci_p;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    note_kernel("pack_filter_kernel");
    const int swz = dtype == DC_F16 ? 1 : 0;  // the fp16 reference layout: rows padded to even, pairs swizzled
    pack_filter_kernel<<<blocks, 256, 0, s>>>((const uint16_t *)filter, (uint16_t *)packed, g.in_c, g.out_c, K2,
                                              swz ? g.out_c + (g.out_c & 1) : g.out_c, ci_p, co_p, swz);
    return hipGetLastError();
}

namespace {

template <typename T, int ITERS>
void dw_launch(dim3 grid, int block, bool eager, hipStream_t s, int act, const ConvP &p, const T *in, const T *filter,
               const T *bias, T *out, const int32_t *mask, int32_t *out_mask, EpiP e, int lg) {
#define DC_DW(A) \
    do { \
        if (p.Kh == 3 && p.Kw == 3 && eager) conv_dw_kernel<T, (ITERS > 2 ? 2 : ITERS), A, true, true><<<grid, block, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg); \
        else if (p.Kh == 3 && p.Kw == 3) conv_dw_kernel<T, ITERS, A, true, false><<<grid, block, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg); \
        else conv_dw_kernel<T, ITERS, A, false, false><<<grid, block, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg); \
    } while (0)
    switch (act) {
        case DC_ACT_LINEAR: DC_DW(DC_ACT_LINEAR); break;
        case DC_ACT_RELU: DC_DW(DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_DW(DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_DW(DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_DW(DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_DW(DC_ACT_SWISH); break;
        default: DC_DW(-1); break;
    }
#undef DC_DW
}

// Depthwise fast path; returns false if the shape does not qualify.
template <typename T>
bool try_depthwise(const dc_geometry &g, const ConvP &p, const T *in, const T *filter,
                   const T *bias, T *out, const int32_t *mask, int32_t *out_mask,
                   const ActEpilogue *epi, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    const auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (g.groups != g.in_c || g.groups != g.out_c || g.groups == 1) return false;
    if (g.in_c % N != 0 || g.kernel_h * g.kernel_w > 64 || g.in_c / N > WAVE * 4) return false;
    if (!al(in) || !al(filter) || !al(out) || (bias && !al(bias))) return false;
    if (epi && (!al(epi->prev) || (epi->trunc && !al(epi->trunc)) || epi->mode < 0)) return false;
    const int64_t P_out = (int64_t)g.batch * g.out_h * g.out_w;
    const int nvec = g.in_c / N;
    // very large maps: mask scan and compaction per wavefront (see conv_dw_scan_kernel)
    // (measured against the strip kernel and the per-pixel kernel on sparse and dense maps: it
    // wins from 2^18 outputs on; with a stride -- where no strip kernel exists -- and with rows of
    // up to 8 vectors, where it serves one pixel per lane group out of LDS-held filters, from 2^16)
    const bool strided = g.stride_h > 1 || g.stride_w > 1;
    if (g.kernel_h == 3 && g.kernel_w == 3 && nvec <= WAVE && P_out >= ((strided || nvec <= 8) ? 1 << 16 : 1 << 18) && P_out < (1ll << 31) &&
        (int64_t)g.batch * g.in_h * g.in_w < (1ll << 31) && g.out_h < 65536 && g.out_w < 65536 &&
        (epi == nullptr || epi->trunc != nullptr)) {
        const int lg = log2i(group_lanes(nvec, 1));
        dim3 grid((unsigned)ceil_div64(P_out, 4 * WAVE));
        EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f, epi ? epi->mode : 0};
        const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
        note_kernel("conv_dw_scan_kernel");
        // up to 8 vectors per pixel: 8 or more pixels per pass already, so one pixel per lane
        // group and the filter in LDS (82 registers, 5 wavefronts per SIMD instead of 2) is
        // 5-25 % faster; wider rows have few pixels per pass and keep two in flight per group
        const bool lean = nvec <= 8;
#define DC_DWN(A)                                                                                                  \
    do {                                                                                                           \
        if (lean) conv_dw_scan_kernel<T, A, 1, true><<<grid, 256, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg); \
        else conv_dw_scan_kernel<T, A, 2, false><<<grid, 256, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg);     \
    } while (0)
        switch (act) {
            case DC_ACT_LINEAR: DC_DWN(DC_ACT_LINEAR); break;
            case DC_ACT_RELU: DC_DWN(DC_ACT_RELU); break;
            case DC_ACT_RELU6: DC_DWN(DC_ACT_RELU6); break;
            case DC_ACT_LEAKY: DC_DWN(DC_ACT_LEAKY); break;
            case DC_ACT_SIGMOID: DC_DWN(DC_ACT_SIGMOID); break;
            case DC_ACT_SWISH: DC_DWN(DC_ACT_SWISH); break;
            default: DC_DWN(-1); break;
        }
#undef DC_DWN
        return true;
    }
    // large maps: strips of four output pixels per group of lanes (see conv_dw_strip_kernel)
    if (g.kernel_h == 3 && g.kernel_w == 3 && g.stride_h == 1 && g.stride_w == 1 && g.dilation_h == 1 &&
        g.dilation_w == 1 && nvec <= WAVE && P_out * g.in_c * (int64_t)sizeof(T) >= (4 << 20)) {
        const int G = group_lanes(nvec, 1);
        const int lg = log2i(G);
        const int64_t strips = (int64_t)g.batch * g.out_h * ceil_div(g.out_w, 4);
        dim3 grid((unsigned)ceil_div64(strips * G, 256));
        EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f, epi ? epi->mode : 0};
        const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
        note_kernel("conv_dw_strip_kernel");
        // filter in LDS (measured): from 8 MB of output on with rows of more than 8 vectors
        const bool lw = nvec > 8 && P_out * g.in_c * (int64_t)sizeof(T) >= (8 << 20);
#define DC_DWS(A)                                                                                              \
    do {                                                                                                       \
        if (lw) conv_dw_strip_kernel<T, A, true><<<grid, 256, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg);   \
        else conv_dw_strip_kernel<T, A, false><<<grid, 256, 0, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg);     \
    } while (0)
        switch (act) {
            case DC_ACT_LINEAR: DC_DWS(DC_ACT_LINEAR); break;
            case DC_ACT_RELU: DC_DWS(DC_ACT_RELU); break;
            case DC_ACT_RELU6: DC_DWS(DC_ACT_RELU6); break;
            case DC_ACT_LEAKY: DC_DWS(DC_ACT_LEAKY); break;
            case DC_ACT_SIGMOID: DC_DWS(DC_ACT_SIGMOID); break;
            case DC_ACT_SWISH: DC_DWS(DC_ACT_SWISH); break;
            default: DC_DWS(-1); break;
        }
#undef DC_DWS
        return true;
    }
    const int wide = (epi == nullptr || epi->mode == DC_TRUNC_MAX) ? wide_group(nvec, P_out) : 0;
    const int G = wide ? wide : pick_group(nvec, P_out, 4);
    const int iters = ceil_div(nvec, G);
    const int block = wide ? wide : group_block(P_out * G);
    note_kernel("conv_dw_kernel");
    dim3 grid((unsigned)ceil_div64(P_out * G, block));
    EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f,
           epi ? epi->mode : 0};
    const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
    const int lg = log2i(G);
    // eager loads where reading nine rows for every pixel, active or not, costs little: maps
    // of up to 2 MB of input, and at most two vectors per lane (register budget)
    const bool eager = iters <= 2 && (int64_t)g.batch * g.in_h * g.in_w * g.in_c * (int64_t)sizeof(T) <= (2 << 20);
    switch (iters) {
        case 1: dw_launch<T, 1>(grid, block, eager, s, act, p, in, filter, bias, out, mask, out_mask, e, lg); break;
        case 2: dw_launch<T, 2>(grid, block, eager, s, act, p, in, filter, bias, out, mask, out_mask, e, lg); break;
        default: dw_launch<T, 4>(grid, block, false, s, act, p, in, filter, bias, out, mask, out_mask, e, lg); break;
    }
    return true;
}

// The depthwise layer that finishes its producer's open activation (conv_dw_kernel<FIN>): 3x3,
// stride 1 or 2, padding 1, on maps small enough for the eager per-pixel form (where launches, not
// bytes, are the cost).  Returns false if the shape does not qualify; nothing is launched then.
template <typename T>
bool try_depthwise_closing(const dc_geometry &g, const ConvP &p, const T *in, const T *filter, T *out,
                           const int32_t *mask, int32_t *out_mask, const ActEpilogue *epi, const OpenAct &open,
                           bool launch, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    const auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (g.groups != g.in_c || g.groups != g.out_c || g.groups == 1) return false;
    if (g.kernel_h != 3 || g.kernel_w != 3 || g.stride_h != g.stride_w || (g.stride_h != 1 && g.stride_h != 2) ||
        g.dilation_h != 1 || g.dilation_w != 1 || g.pad_top != 1 || g.pad_left != 1 || g.pad_bottom != 1 ||
        g.pad_right != 1)
        return false;
    // (stride 2: every input pixel lies in the 2 x 2 block of exactly one output pixel)
    if (g.stride_h == 2 && (2 * g.out_h < g.in_h || 2 * g.out_w < g.in_w)) return false;
    if (g.in_c % N != 0 || g.in_c / N > WAVE * 4) return false;
    if (epi == nullptr || epi->trunc == nullptr || epi->mode < 0) return false;
    const int64_t P_out = (int64_t)g.batch * g.out_h * g.out_w;
    const int nvec = g.in_c / N;
    if (P_out >= (1 << 16) || P_out * g.in_c * (int64_t)sizeof(T) >= (4 << 20)) return false;  // scan / strip kernels
    const int wide = epi->mode == DC_TRUNC_MAX ? wide_group(nvec, P_out) : 0;
    const int G = wide ? wide : pick_group(nvec, P_out, 4);
    const int iters = ceil_div(nvec, G);
    // the eager form only (its input at most 2 MB); stride 2: one vector per lane, the state of four pixels
    if (iters > (g.stride_h == 2 ? 1 : 2) || (int64_t)g.batch * g.in_h * g.in_w * g.in_c * (int64_t)sizeof(T) > (2 << 20))
        return false;
    if (!launch) return true;
    if (!al(in) || !al(filter) || !al(out) || !al(epi->prev) || !al(epi->trunc) || !al(open.prev) || !al(open.trunc))
        return false;
    const int block = wide ? wide : group_block(P_out * G);
    note_kernel("conv_dw_kernel");
    dim3 grid((unsigned)ceil_div64(P_out * G, block));
    EpiP e{epi->prev, epi->trunc, epi->thr, epi->mode};
    OpenActP f{open.prev, open.trunc, open.thr};
    const int act = epi->act < 0 ? 0 : epi->act;
    const int lg = log2i(G);
#define DC_DWF(A)                                                                                                      \
    do {                                                                                                               \
        if (g.stride_h == 2) conv_dw_kernel<T, 1, A, true, true, 2><<<grid, block, 0, s>>>(p, in, filter, nullptr, out, mask, out_mask, e, lg, f); \
        else if (iters == 1) conv_dw_kernel<T, 1, A, true, true, 1><<<grid, block, 0, s>>>(p, in, filter, nullptr, out, mask, out_mask, e, lg, f); \
        else conv_dw_kernel<T, 2, A, true, true, 1><<<grid, block, 0, s>>>(p, in, filter, nullptr, out, mask, out_mask, e, lg, f); \
    } while (0)
    switch (act) {
        case DC_ACT_RELU: DC_DWF(DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_DWF(DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_DWF(DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_DWF(DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_DWF(DC_ACT_SWISH); break;
        default: DC_DWF(DC_ACT_LINEAR); break;
    }
#undef DC_DWF
    return true;
}

// Stems of large frames on the matrix cores (see conv_stem_mfma_kernel); false if the shape, the
// operands' alignment or the map size do not qualify.
template <typename E>
bool try_stem_mfma(const dc_geometry &g, const ConvP &p, const E *in, const E *packed,
                   const E *bias, E *out, const int32_t *mask, int32_t *out_mask,
                   const ActEpilogue *epi, hipStream_t s) {
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    if (packed == nullptr || !stem_eligible(g, DC_F16)) return false;
    // many channel tiles on a large map: the per-pixel kernel's wide stores win (measured)
    if (g.out_c > 32 && (int64_t)g.batch * g.out_h * g.out_w > 65536) return false;
    if (!al8(out) || (bias && !al8(bias)) || (reinterpret_cast<uintptr_t>(packed) & 15u) != 0) return false;
    if (epi && (epi->mode < 0 || epi->trunc == nullptr || !al8(epi->prev) || !al8(epi->trunc))) return false;
    const int hal_h = (TILE - 1) * g.stride_h + g.kernel_h;
    const int hal_wp = (TILE - 1) * g.stride_w + STEM_K;  // every lane reads 8 window columns
    const size_t lds = (size_t)hal_h * hal_wp * 8 + (size_t)hal_h * 4;
    dim3 grid(ceil_div(g.out_w, TILE), ceil_div(g.out_h, TILE), g.batch);
    EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f, epi ? epi->mode : 0};
    const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
    const int co_tiles = ceil_div(g.out_c, 16);
    // maps of 2^18 pixels and more: only updated pixels and the filters of updated tiles are read
    const int lazy = (int64_t)g.batch * g.in_h * g.in_w >= (1 << 18) ? 1 : 0;
    note_kernel("conv_stem_mfma_kernel");
#define DC_ST_R(A)                                                                                                   \
    do {                                                                                                             \
        if (co_tiles == 1) conv_stem_mfma_kernel<E, 1, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_wp, lazy); \
        else if (co_tiles == 2) conv_stem_mfma_kernel<E, 2, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_wp, lazy); \
        else conv_stem_mfma_kernel<E, 4, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_wp, lazy); \
    } while (0)
    switch (act) {
        case DC_ACT_LINEAR: DC_ST_R(DC_ACT_LINEAR); break;
        case DC_ACT_RELU: DC_ST_R(DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_ST_R(DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_ST_R(DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_ST_R(DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_ST_R(DC_ACT_SWISH); break;
        default: DC_ST_R(-1); break;
    }
#undef DC_ST_R
    return true;
}

// Shapes conv_thin_mfma_kernel takes (16-bit types).
inline bool thin_shape(const dc_geometry &g) {
    return g.groups == 1 && (g.in_c == 8 || g.in_c == 16) && g.kernel_h <= 3 && g.kernel_w <= 3 &&
           g.kernel_h * g.kernel_w >= 2 && g.dilation_h == 1 && g.dilation_w == 1 && g.stride_h <= 2 && g.stride_w <= 2 &&
           g.out_c % 8 == 0 && g.out_c <= 64 &&
           (int64_t)g.batch * g.out_h * g.out_w >= 32768 &&  // small maps: latency, not bandwidth, is the cost
           !patch_eligible(g, DC_F16);                       // ... and the 4x4-patch kernel's layers stay with it
}

// Thin K x K layers of large maps on the matrix cores (see conv_thin_mfma_kernel).  Returns 0 if
// the shape, the operands' alignment or the map size do not qualify (nothing launched), 1 if the
// layer is done, 2 if the convolution is done and the caller has to launch the activation /
// truncation `epi` describes (anything but the maximum norm): the layer keeps this kernel's
// summation order whatever follows it.
template <typename E>
int try_thin_mfma(const dc_geometry &g, const ConvP &p, const E *in, const E *packed, const E *bias, E *out,
                  const int32_t *mask, int32_t *out_mask, const ActEpilogue *epi, hipStream_t s) {
    const auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (packed == nullptr || !thin_shape(g)) return 0;
    if (!al16(in) || !al16(out) || !al16(packed) || (bias && (reinterpret_cast<uintptr_t>(bias) & 7u) != 0)) return 0;
    const ActEpilogue *pending = nullptr;
    if (epi && (epi->mode != DC_TRUNC_MAX || epi->trunc == nullptr || !al16(epi->prev) || !al16(epi->trunc))) {
        pending = epi;
        epi = nullptr;
    }
    const int hal_h = (TILE - 1) * g.stride_h + g.kernel_h, hal_w = (TILE - 1) * g.stride_w + g.kernel_w;
    const int co_tiles = ceil_div(g.out_c, 16);
    const int R = co_tiles <= 1 ? 1 : co_tiles <= 2 ? 2 : 4;
    const size_t lds = (size_t)hal_h * hal_w * g.in_c * 2 + (size_t)4 * 16 * (R * 32 + 16) + (size_t)hal_h * 4;
    dim3 grid(ceil_div(g.out_w, TILE), ceil_div(g.out_h, TILE), g.batch);
    EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f, epi ? epi->mode : 0};
    const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
    const int lazy = (int64_t)g.batch * g.in_h * g.in_w >= (1 << 18) ? 1 : 0;
    note_kernel("conv_thin_mfma_kernel");
#define DC_TH_R(CI, M, A)                                                                                            \
    do {                                                                                                             \
        if (R == 1) conv_thin_mfma_kernel<E, CI, 1, M, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_w, lazy); \
        else if (R == 2) conv_thin_mfma_kernel<E, CI, 2, M, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_w, lazy); \
        else conv_thin_mfma_kernel<E, CI, 4, M, A><<<grid, 256, lds, s>>>(p, in, packed, bias, out, mask, out_mask, e, hal_h, hal_w, lazy); \
    } while (0)
#define DC_TH(M, A)                                                                                                  \
    do {                                                                                                             \
        if (g.in_c == 16) DC_TH_R(16, M, A); else DC_TH_R(8, M, A);                                                  \
    } while (0)
    switch (act) {
        case DC_ACT_LINEAR: DC_TH(2, DC_ACT_LINEAR); break;
        case DC_ACT_RELU: DC_TH(2, DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_TH(2, DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_TH(2, DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_TH(2, DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_TH(2, DC_ACT_SWISH); break;
        default: DC_TH(0, 0); break;
    }
#undef DC_TH
#undef DC_TH_R
    return pending != nullptr ? 2 : 1;
}

template <typename T>
bool try_fewcin(const dc_geometry &g, const ConvP &p, const T *in, const T *filter, const T *bias,
                T *out, const int32_t *mask, int32_t *out_mask, const ActEpilogue *epi,
                hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    const auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (g.groups != 1 || g.in_c > 4 || g.out_c % N != 0 || g.out_c / N > WAVE) return false;
    if (g.kernel_h * g.kernel_w > 64) return false;
    if (!al(filter) || !al(out) || (bias && !al(bias))) return false;
    if (epi && (!al(epi->prev) || (epi->trunc && !al(epi->trunc)) || epi->mode < 0)) return false;
    const int64_t P_out = (int64_t)g.batch * g.out_h * g.out_w;
    const int G = group_lanes(g.out_c / N, 1);
    const int block = group_block(P_out * G);
    dim3 grid((unsigned)ceil_div64(P_out * G, block));
    EpiP e{epi ? epi->prev : nullptr, epi ? epi->trunc : nullptr, epi ? epi->thr : 0.f,
           epi ? epi->mode : 0};
    const int act = epi ? (epi->act < 0 ? 0 : epi->act) : -1;
    const int lg = log2i(G);
    note_kernel("conv_fewcin_kernel");
    const bool k3 = g.kernel_h == 3 && g.kernel_w == 3;
    // the un-swizzled filter goes to LDS when it fits (always for 3x3)
    const size_t fbytes = (size_t)g.kernel_h * g.kernel_w * g.in_c * g.out_c * sizeof(T);
    const int staged = !k3 && fbytes <= (32 << 10) ? 1 : 0;
    const size_t lds = (k3 || staged) ? fbytes : 0;
#define DC_FC(A)                                                                                              \
    do {                                                                                                      \
        if (k3) conv_fewcin_kernel<T, A, true><<<grid, block, lds, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg, 0); \
        else conv_fewcin_kernel<T, A, false><<<grid, block, lds, s>>>(p, in, filter, bias, out, mask, out_mask, e, lg, staged); \
    } while (0)
    switch (act) {
        case DC_ACT_LINEAR: DC_FC(DC_ACT_LINEAR); break;
        case DC_ACT_RELU: DC_FC(DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_FC(DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_FC(DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_FC(DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_FC(DC_ACT_SWISH); break;
        default: DC_FC(-1); break;
    }
#undef DC_FC
    return true;
}

}  // namespace

// The filter is re-read by every patch, so the patch kernel only pays while
// patches x channel tiles x reduction steps stays small.
bool patch_eligible(const dc_geometry &g, int dtype) {
    if (!mfma_eligible(g, dtype) || g.kernel_h * g.kernel_w > MFMA_MAX_TAPS) return false;
    const int64_t patches = (int64_t)ceil_div(g.out_w, 4) * ceil_div(g.out_h, 4) * g.batch;
    const int steps = g.kernel_h * g.kernel_w * (round_up(g.in_c, 32) / 32);
    return patches * ceil_div(g.out_c, 16) * steps <= 32768;
}

namespace {
// Launch plan of conv_lds_mfma_kernel for a layer the 4x4-patch kernel does not take; !ok: the
// halo or the step table does not fit (or a transposed convolution is dilated).
struct LdsPlan {
    bool ok;
    int hal_h, hal_w, ltx, lty, vk2, kcc, rl, ksl, ncw;
};

LdsPlan lds_plan(const dc_geometry &g, bool transposed) {
    LdsPlan lp{};
    if (transposed && !(g.dilation_h == 1 && g.dilation_w == 1)) return lp;
    const int co_tiles = ceil_div(g.out_c, 16);
    const int ksteps_all = round_up(g.in_c, 32) / 32;
    // taps per dimension seen by a tile: all of them, or those of one stride phase
    const int vkh = transposed ? ceil_div(g.kernel_h, g.stride_h) : g.kernel_h;
    const int vkw = transposed ? ceil_div(g.kernel_w, g.stride_w) : g.kernel_w;
    lp.vk2 = vkh * vkw;
    lp.hal_h = transposed ? TILE + vkh - 1 : (TILE - 1) * g.stride_h + (g.kernel_h - 1) * g.dilation_h + 1;
    lp.hal_w = transposed ? TILE + vkw - 1 : (TILE - 1) * g.stride_w + (g.kernel_w - 1) * g.dilation_w + 1;
    // transposed: one tile per (8x8 block of pixels one stride apart, stride phase)
    lp.ltx = transposed ? ceil_div(ceil_div(g.out_w, g.stride_w), TILE) * g.stride_w : ceil_div(g.out_w, TILE);
    lp.lty = transposed ? ceil_div(ceil_div(g.out_h, g.stride_h), TILE) * g.stride_h : ceil_div(g.out_h, TILE);
    const int hpx = lp.hal_h * lp.hal_w;
    // Arrangements (R channel tiles per wavefront, KS reduction slices, channel groups):
    // wide outputs on many tiles: R = 2, four channel groups; otherwise, with enough
    // steps to split, R = 2 and two or four slices (x two or one channel groups); short
    // reductions: R = 1, up to four channel groups.
    const int64_t tiles = (int64_t)lp.ltx * lp.lty * g.batch;
    auto plan = [&](int lds_budget) {
        const int kmax = hpx <= LDS_MAX_HALO ? (lds_budget / hpx - 16) / 64 : 0;
        lp.kcc = kmax >= 1 ? ceil_div(ksteps_all, ceil_div(ksteps_all, kmax)) : 0;
        const int nsteps_chunk = lp.vk2 * lp.kcc;
        lp.rl = 1; lp.ksl = 1; lp.ncw = std::min(4, co_tiles);
        if (co_tiles >= 16 && tiles * ceil_div(co_tiles, 8) >= 512) { lp.rl = 2; lp.ncw = 4; }
        else if (nsteps_chunk >= 36 && co_tiles >= 4 && tiles * ceil_div(co_tiles, 4) < 128) {
            // very few tiles (deep layers on small maps): one channel group per workgroup doubles
            // the workgroups and halves the filter bytes each streams (measured: 512 -> 512 on
            // 17 x 30, 14.5 -> 13.3 us)
            lp.rl = 2; lp.ksl = 4; lp.ncw = 1;
        }
        else if (nsteps_chunk >= 16 && co_tiles >= 4) {
            // no more workgroups than compute units and a long reduction: eight wavefronts
            lp.rl = 2; lp.ncw = 2;
            lp.ksl = (nsteps_chunk >= 36 && tiles * ceil_div(co_tiles, 4) <= 256) ? 4 : 2;
        }
        else if (nsteps_chunk >= 16 && co_tiles >= 2) { lp.rl = 2; lp.ksl = 4; lp.ncw = 1; }
    };
    // Fewer LDS passes over the input channels (each costs a table, a staging round trip
    // and a ring start-up) where a larger halo does not cost residency: a compute unit
    // holds one workgroup of this launch anyway.  Otherwise 48 KB, two workgroups per
    // compute unit.
    plan(48 << 10);
    const int passes_small = lp.kcc >= 1 ? ceil_div(ksteps_all, lp.kcc) : 1 << 30;
    plan(112 << 10);
    if (!(lp.kcc >= 1 && ceil_div(ksteps_all, lp.kcc) < passes_small &&
          tiles * ceil_div(co_tiles, lp.ncw * lp.rl) <= 256))
        plan(48 << 10);
    // the step table holds all steps of a channel chunk plus the ring's run-out
    lp.ok = lp.kcc >= 1 && lp.vk2 * lp.kcc + 48 <= LDS_MAX_STEPS;
    return lp;
}

// res != nullptr (plain convolutions only): the DCAdd behind the convolution runs on the
// accumulators, see conv_lds_mfma_kernel.
// Can the layer's activation / truncation be finished in the convolution's launch?  One workgroup
// holds all channels of its pixels, rows of 16-byte vectors, at most two per lane of a wavefront,
// and no more workgroups than compute units (see LdsFin).
bool lds_finishes_activation(const dc_geometry &g, const LdsPlan &lp, bool transposed, const Residual *res,
                             const void *out, const ActEpilogue *epi) {
    const auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (epi == nullptr || transposed || res != nullptr || epi->mode < 0 || epi->trunc == nullptr || epi->prev == nullptr)
        return false;
    if (epi->act != DC_ACT_LINEAR && epi->act != DC_ACT_RELU && epi->act != DC_ACT_RELU6 && epi->act != DC_ACT_LEAKY)
        return false;
    if (g.out_c % 8 != 0 || g.out_c > 1024 || !al16(epi->prev) || !al16(epi->trunc) || !al16(out)) return false;
    return ceil_div(ceil_div(g.out_c, 16), lp.ncw * lp.rl) == 1 && (int64_t)lp.ltx * lp.lty * g.batch <= 256;
}

// epi + fused: the layer's activation / truncation, finished in this launch where
// lds_finishes_activation allows (then *fused = true), else left to the caller.
template <typename E>
hipError_t launch_lds_conv(const dc_geometry &g, const ConvP &p, const LdsPlan &lp, const void *in, const void *packed,
                           const void *bias, void *out, const int32_t *mask, int32_t *out_mask, bool transposed,
                           const Residual *res, hipStream_t s, const ActEpilogue *epi = nullptr,
                           bool *fused = nullptr) {
    const int co_tiles = ceil_div(g.out_c, 16);
    const int ci_p = round_up(g.in_c, 32);
    const int hpx = lp.hal_h * lp.hal_w;
    const int kcc = lp.kcc, hal_h = lp.hal_h, hal_w = lp.hal_w;
    const int nwv = lp.ncw * lp.ksl;  // wavefronts per workgroup
    const int cbl = ceil_div(co_tiles, lp.ncw * lp.rl);
    size_t lds = std::max((size_t)hpx * (kcc * 64 + 16), lp.ksl > 1 ? (size_t)lp.ksl * lp.ncw * lp.rl * 4 * 1024 : 0);
    const int lgv = log2i(pow2_ceil(kcc * 4));  // lanes per halo pixel while staging
    dim3 lgrid(lp.ltx, lp.lty, g.batch * cbl);
    PatchRes<E> rs{nullptr, nullptr, nullptr, 0.f, 0.f, 0};
    if (res != nullptr) rs = PatchRes<E>{(const E *)res->values, res->mask, (E *)res->prev, res->wa, res->wb, res->act};
    const bool fin = fused != nullptr && lds_finishes_activation(g, lp, transposed, res, out, epi);
    if (fused != nullptr) *fused = fin;
    LdsFin<E> lf{nullptr, nullptr, 0.f, 0, 0, 0, 1};
    if (fin) {
        const int nvec = g.out_c / 8;
        const int iters = nvec > WAVE ? 2 : 1;
        lf = LdsFin<E>{(E *)epi->prev, (E *)epi->trunc, epi->thr, epi->mode, epi->act,
                       log2i(pow2_ceil(ceil_div(nvec, iters))), iters};
        // the tile's sums as pixel rows behind the partial sums of the reduction slices
        lds = std::max(lds, (lp.ksl > 1 ? (size_t)lp.ksl * lp.ncw * lp.rl * 4 * 1024 : 0) +
                                (size_t)TILE_PX * (g.out_c * 2 + 16));
    }
    note_kernel("conv_lds_mfma_kernel");
#define DC_LDS_ARGS (p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, cbl, ci_p, hal_h, hal_w, kcc, lgv, rs, lf)
#define DC_LDS_K(RV, SV, DV, KV, TV, AV, FV)                                                                \
    do {                                                                                                    \
        if (lds > (48u << 10)) {                                                                            \
            const hipError_t big = allow_large_lds(&conv_lds_mfma_kernel<E, RV, SV, DV, KV, TV, AV, FV>);   \
            if (big != hipSuccess) return big;                                                              \
        }                                                                                                   \
        conv_lds_mfma_kernel<E, RV, SV, DV, KV, TV, AV, FV><<<lgrid, nwv * WAVE, lds, s>>> DC_LDS_ARGS;      \
    } while (0)
#define DC_LDS_L(RV, SV, DV, KV)                                                                            \
    do {                                                                                                    \
        if (res != nullptr && transposed) DC_LDS_K(RV, SV, DV, KV, true, true, false);                      \
        else if (res != nullptr) DC_LDS_K(RV, SV, DV, KV, false, true, false);                              \
        else if (transposed) DC_LDS_K(RV, SV, DV, KV, true, false, false);                                  \
        else if (fin) DC_LDS_K(RV, SV, DV, KV, false, false, true);                                         \
        else DC_LDS_K(RV, SV, DV, KV, false, false, false);                                                 \
    } while (0)
    if (lp.rl == 1) DC_LDS_L(1, 2, 3, 1);
    else if (lp.ksl == 1) DC_LDS_L(2, 2, 3, 1);
    else if (lp.ksl == 2) DC_LDS_L(2, 2, 3, 2);
    else DC_LDS_L(2, 2, 3, 4);
#undef DC_LDS_L
#undef DC_LDS_K
#undef DC_LDS_ARGS
    return hipGetLastError();
}
}  // namespace

namespace {
// Arrangement of conv_patch_mfma_kernel for a layer: reduction slices (wavefronts), channel tiles
// per wavefront, channel blocks.
struct PatchPlan {
    int kwv, rv, cbk;
};

PatchPlan patch_plan(const dc_geometry &g) {
    const int co_tiles = ceil_div(g.out_c, 16);
    const int steps = g.kernel_h * g.kernel_w * (round_up(g.in_c, 32) / 32);
    const int64_t patches = (int64_t)ceil_div(g.out_w, 4) * ceil_div(g.out_h, 4) * g.batch;
    PatchPlan pp;
    pp.kwv = steps <= 12 ? 1 : steps <= 48 ? 4 : 8;
    // Two channel tiles per wavefront (they are independent: the summation order of an output does
    // not depend on it) halve the workgroups and the input reads: on many patches; for reductions
    // split over wavefronts while a workgroup's filter slice stays below 40 KB (measured on 64 -> 64
    // ... 256, 64 .. 1024 patches: 4.4 - 4.6 -> 3.7 - 3.9 us; with 128 input channels it loses); and
    // where it puts all channels of a 32-channel layer into one wavefront, which can then finish
    // the layer's activation itself (3.8 + 2.0 -> 4.4 us; without an activation it costs 0.3 us).
    pp.rv = 1;
    if (co_tiles >= 2 && (patches * co_tiles >= 512 || (pp.kwv >= 4 && g.in_c <= 64) || (pp.kwv == 1 && co_tiles == 2)))
        pp.rv = 2;
    pp.cbk = ceil_div(co_tiles, pp.rv);
    return pp;
}

// activation + truncation inside the kernel where one wavefront holds all channels of a pixel
bool patch_fuses_activation(const dc_geometry &g, const PatchPlan &pp, const void *bias, const void *out,
                            const ActEpilogue *epi) {
    const auto al8 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 7u) == 0; };
    return epi != nullptr && pp.kwv == 1 && pp.cbk == 1 && epi->mode >= 0 && epi->trunc != nullptr && g.out_c % 4 == 0 &&
           al8(epi->prev) && al8(epi->trunc) && al8(out) && (bias == nullptr || al8(bias));
}

template <typename E>
hipError_t launch_patch_conv_t(const dc_geometry &g, const void *in, const void *packed,
                               const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                               bool transposed, const Residual *res, hipStream_t s,
                               const ActEpilogue *epi, bool *epilogue_done) {
    ConvP p = make_params(g, DC_F16);  // the packed filter's layout does not depend on the type
    const int ci_p = round_up(g.in_c, 32);
    const PatchPlan pp = patch_plan(g);
    const int kwv = pp.kwv, rv = pp.rv, cbk = pp.cbk;
    dim3 pgrid(ceil_div(g.out_w, 4), ceil_div(g.out_h, 4), g.batch * cbk);
    PatchRes<E> rs{nullptr, nullptr, nullptr, 0.f, 0.f, 0};
    if (res != nullptr)
        rs = PatchRes<E>{(const E *)res->values, res->mask, (E *)res->prev, res->wa, res->wb, res->act};
    const bool k3 = g.kernel_h == 3 && g.kernel_w == 3;
    const bool fuse = epilogue_done != nullptr && res == nullptr && !transposed && patch_fuses_activation(g, pp, bias, out, epi);
    if (epilogue_done != nullptr) *epilogue_done = fuse;
    PatchEpi<E> pe{nullptr, nullptr, 0.f, 0, 0};
    if (fuse) pe = PatchEpi<E>{(E *)epi->prev, (E *)epi->trunc, epi->thr, epi->mode, epi->act < 0 ? 0 : epi->act};
    note_kernel("conv_patch_mfma_kernel");
#define DC_PATCH_ARGS (p, (const E *)in, (const E *)packed, (const E *)bias, (E *)out, mask, out_mask, cbk, ci_p, rs, pe)
#define DC_PATCH_L(TRF, KWV, RV, SV, AV)                                                                      \
    do {                                                                                                      \
        if (k3) conv_patch_mfma_kernel<E, TRF, KWV, RV, SV, AV, true><<<pgrid, KWV * WAVE, 0, s>>> DC_PATCH_ARGS; \
        else conv_patch_mfma_kernel<E, TRF, KWV, RV, SV, AV, false><<<pgrid, KWV * WAVE, 0, s>>> DC_PATCH_ARGS;  \
    } while (0)
#define DC_PATCH(TRF, AV)                                                                       \
    do {                                                                                        \
        if (kwv == 1) { if (rv == 2) DC_PATCH_L(TRF, 1, 2, 9, AV); else DC_PATCH_L(TRF, 1, 1, 9, AV); } \
        else if (kwv == 4) { if (rv == 2) DC_PATCH_L(TRF, 4, 2, 5, AV); else DC_PATCH_L(TRF, 4, 1, 9, AV); } \
        else { if (rv == 2) DC_PATCH_L(TRF, 8, 2, 6, AV); else DC_PATCH_L(TRF, 8, 1, 9, AV); } \
    } while (0)
    if (res != nullptr) DC_PATCH(false, 1);  // the fused sum exists for plain convolutions only
    else if (transposed) DC_PATCH(true, 0);
    else if (fuse) { if (rv == 2) DC_PATCH_L(false, 1, 2, 9, 2); else DC_PATCH_L(false, 1, 1, 9, 2); }
    else DC_PATCH(false, 0);
#undef DC_PATCH
#undef DC_PATCH_L
#undef DC_PATCH_ARGS
    return hipGetLastError();
}
}  // namespace

// Layers of the LDS-halo kernel (larger K x K convolutions, plain or transposed) have the fused
// residual sum too, for a DCAdd without activation.
bool lds_add_eligible(const dc_geometry &g, int dtype, int activation, bool transposed) {
    // transposed: every stride phase of the output needs at least one tap (window >= stride), so
    // that every output tile runs the reduction kernel's epilogue
    if (transposed && (g.kernel_h < g.stride_h || g.kernel_w < g.stride_w)) return false;
    // a layer of the thin-layer kernel keeps that kernel's summation order: no fused sum
    if (!transposed && thin_shape(g)) return false;
    return activation <= 0 && mfma_eligible(g, dtype) && g.kernel_h * g.kernel_w <= MFMA_MAX_TAPS && !patch_eligible(g, dtype) &&
           lds_plan(g, transposed).ok;
}

hipError_t launch_lds_conv_add(const dc_geometry &g, const void *in, const void *packed, const void *bias,
                               void *out, const int32_t *mask, int32_t *out_mask, const Residual *res,
                               int dtype, hipStream_t s, bool transposed) {
    const ConvP p = make_params(g, DC_F16);  // the packed filter's layout does not depend on the type
    const LdsPlan lp = lds_plan(g, transposed);
    if (dtype == DC_BF16) return launch_lds_conv<bf16_t>(g, p, lp, in, packed, bias, out, mask, out_mask, transposed, res, s);
    return launch_lds_conv<half_t>(g, p, lp, in, packed, bias, out, mask, out_mask, transposed, res, s);
}

hipError_t launch_patch_conv(const dc_geometry &g, const void *in, const void *packed,
                             const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                             bool transposed, const Residual *res, int dtype, hipStream_t s,
                             const ActEpilogue *epi, bool *epilogue_done) {
    if (dtype == DC_BF16)
        return launch_patch_conv_t<bf16_t>(g, in, packed, bias, out, mask, out_mask, transposed, res, s, epi, epilogue_done);
    return launch_patch_conv_t<half_t>(g, in, packed, bias, out, mask, out_mask, transposed, res, s, epi, epilogue_done);
}

// Layers launch_conv / dc_conv_add route to conv_patch_mfma_kernel and the group launch can hold.
bool conv_group_item_eligible(const ConvGroupItem &c, int dtype) {
    const dc_geometry &g = c.g;
    return c.packed != nullptr && g.kernel_h == 3 && g.kernel_w == 3 && !pointwise_eligible(g, dtype) &&
           patch_eligible(g, dtype) && !(c.res != nullptr && c.epi != nullptr);
}

bool conv_group_activation_fused(const ConvGroupItem &c) {
    return c.res == nullptr && patch_fuses_activation(c.g, patch_plan(c.g), c.bias, c.out, c.epi);
}

namespace {
template <typename E>
hipError_t launch_conv_group_t(const ConvGroupItem *items, int n, hipStream_t s) {
    PatchGroup<E> pg;
    pg.n = n;
    int blocks = 0, kmax = 1;
    // Workgroups start in grid order: the layers whose workgroups stream the most filter (a
    // reduction split over eight wavefronts) go first, so that the short ones fill in behind
    // them rather than delay them (measured on four branches: 10.7 -> 9.7 us; sorting all layers
    // by reduction length costs the two- and three-branch groups 0.5 us).
    int order[GROUP_MAX];
    for (int i = 0; i < n; ++i) order[i] = i;
    std::stable_sort(order, order + n, [&](int a, int b) { return (patch_plan(items[a].g).kwv == 8) > (patch_plan(items[b].g).kwv == 8); });
    for (int i = 0; i < n; ++i) {
        const ConvGroupItem &c = items[order[i]];
        const dc_geometry &g = c.g;
        PatchItem<E> &it = pg.it[i];
        const PatchPlan pp = patch_plan(g);
        it.p = make_params(g, DC_F16);
        it.in = (const E *)c.in; it.wp = (const E *)c.packed; it.bias = (const E *)c.bias;
        it.out = (E *)c.out; it.mask = c.mask; it.out_mask = c.out_mask;
        it.co_blocks = pp.cbk; it.ci_p = round_up(g.in_c, 32);
        it.rs = PatchRes<E>{nullptr, nullptr, nullptr, 0.f, 0.f, 0};
        it.ep = PatchEpi<E>{nullptr, nullptr, 0.f, 0, 0};
        it.mode = 0;
        if (c.res != nullptr) {
            it.rs = PatchRes<E>{(const E *)c.res->values, c.res->mask, (E *)c.res->prev, c.res->wa, c.res->wb, c.res->act};
            it.mode = 1;
        } else if (conv_group_activation_fused(c)) {
            it.ep = PatchEpi<E>{(E *)c.epi->prev, (E *)c.epi->trunc, c.epi->thr, c.epi->mode, c.epi->act < 0 ? 0 : c.epi->act};
            it.mode = 2;
        }
        it.kwv = pp.kwv; it.rv = pp.rv;
        it.gx = ceil_div(g.out_w, 4); it.gy = ceil_div(g.out_h, 4);
        it.first = blocks;
        blocks += it.gx * it.gy * g.batch * pp.cbk;
        kmax = std::max(kmax, pp.kwv);
    }
    for (int i = n; i < GROUP_MAX; ++i) pg.it[i] = pg.it[0];
    note_kernel("conv_patch_group_kernel");
    conv_patch_group_kernel<E><<<dim3((unsigned)blocks), kmax * WAVE, 0, s>>>(pg);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_conv_group(const ConvGroupItem *items, int n, int dtype, hipStream_t s) {
    if (dtype == DC_BF16) return launch_conv_group_t<bf16_t>(items, n, s);
    return launch_conv_group_t<half_t>(items, n, s);
}

namespace {
// E16: the 16-bit element type of the matrix-core paths (half_t where dtype is fp32 -- those
// paths are not eligible then).
template <typename E16>
hipError_t launch_conv_t(const dc_geometry &g, const void *in, const void *filter,
                         const void *packed, const void *bias, void *out, const int32_t *mask,
                         int32_t *out_mask, int dtype, bool transposed, const ActEpilogue *epi,
                         hipStream_t s) {
    ConvP p = make_params(g, dtype);
    const int tx = ceil_div(g.out_w, TILE), ty = ceil_div(g.out_h, TILE);
    if (!transposed) {
        const bool done = dtype == DC_F32
            ? try_depthwise<float>(g, p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, epi, s)
            : dtype == DC_BF16
            ? try_depthwise<bf16_t>(g, p, (const bf16_t *)in, (const bf16_t *)filter, (const bf16_t *)bias, (bf16_t *)out, mask, out_mask, epi, s)
            : try_depthwise<half_t>(g, p, (const half_t *)in, (const half_t *)filter, (const half_t *)bias, (half_t *)out, mask, out_mask, epi, s);
        if (done) return hipGetLastError();
        if (dtype != DC_F32 && try_stem_mfma<E16>(g, p, (const E16 *)in, (const E16 *)packed, (const E16 *)bias,
                                                  (E16 *)out, mask, out_mask, epi, s))
            return hipGetLastError();
        const int thin = dtype == DC_F32 ? 0 : try_thin_mfma<E16>(g, p, (const E16 *)in, (const E16 *)packed, (const E16 *)bias,
                                                                  (E16 *)out, mask, out_mask, epi, s);
        if (thin != 0) {
            const hipError_t te = hipGetLastError();
            if (te != hipSuccess || thin == 1) return te;
            return launch_activate_truncate(out, epi->prev, epi->trunc, out_mask, epi->thr, epi->act,
                                            epi->mode, g.batch * g.out_h * g.out_w, g.out_c, dtype, s);
        }
        const bool few = dtype == DC_F32
            ? try_fewcin<float>(g, p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, epi, s)
            : dtype == DC_BF16
            ? try_fewcin<bf16_t>(g, p, (const bf16_t *)in, (const bf16_t *)filter, (const bf16_t *)bias, (bf16_t *)out, mask, out_mask, epi, s)
            : try_fewcin<half_t>(g, p, (const half_t *)in, (const half_t *)filter, (const half_t *)bias, (half_t *)out, mask, out_mask, epi, s);
        if (few) return hipGetLastError();
    }
    if (packed != nullptr && !transposed && pointwise_eligible(g, dtype)) {
        bool epilogue_done = false;
        hipError_t e = launch_pointwise(g, in, packed, bias, out, mask, out_mask, epi, &epilogue_done, nullptr, dtype, s);
        if (e != hipSuccess || epi == nullptr || epilogue_done) return e;
        return launch_activate_truncate(out, epi->prev, epi->trunc, out_mask, epi->thr, epi->act,
                                        epi->mode, g.batch * g.out_h * g.out_w, g.out_c, dtype, s);
    }
    if (packed != nullptr && mfma_eligible(g, dtype) && g.kernel_h * g.kernel_w <= MFMA_MAX_TAPS) {
        const int co_tiles = ceil_div(g.out_c, 16);
        const int ci_p = round_up(g.in_c, 32);
        const int steps = g.kernel_h * g.kernel_w * (ci_p / 32);
        // Small layers: one 4x4 output patch per workgroup (see conv_patch_mfma_kernel).
        if (patch_eligible(g, dtype)) {
            bool fused = false;
            hipError_t pe = launch_patch_conv_t<E16>(g, in, packed, bias, out, mask, out_mask, transposed, nullptr, s, epi, &fused);
            if (pe != hipSuccess || epi == nullptr || fused) return pe;
            return launch_activate_truncate(out, epi->prev, epi->trunc, out_mask, epi->thr, epi->act,
                                            epi->mode, g.batch * g.out_h * g.out_w, g.out_c, dtype, s);
        }
        // Larger layers: halo staged in LDS (see conv_lds_mfma_kernel).
        const LdsPlan lp = lds_plan(g, transposed);
        if (lp.ok) {
            // thin layers on large maps: the filter stays in registers while a workgroup walks over tiles
            const bool resident = !transposed &&
                resident_conv_eligible(g, lp.hal_h, lp.hal_w, lp.ltx, lp.lty, lp.kcc, lp.rl, lp.ksl, lp.ncw);
            bool fused = false;
            hipError_t le = resident
                ? launch_resident_conv(g, p, lp.hal_h, lp.hal_w, lp.ltx, lp.lty, lp.kcc, lp.rl, lp.ksl, lp.ncw, in, packed,
                                       bias, out, mask, out_mask, dtype, s)
                : launch_lds_conv<E16>(g, p, lp, in, packed, bias, out, mask, out_mask, transposed, nullptr, s, epi, &fused);
            if (le != hipSuccess || epi == nullptr || fused) return le;
            return launch_activate_truncate(out, epi->prev, epi->trunc, out_mask, epi->thr, epi->act,
                                            epi->mode, g.batch * g.out_h * g.out_w, g.out_c, dtype, s);
        }
        // transposed: one tile per (8x8 block of pixels one stride apart, stride phase)
        const int gtx = transposed ? ceil_div(ceil_div(g.out_w, g.stride_w), TILE) * g.stride_w : tx;
        const int gty = transposed ? ceil_div(ceil_div(g.out_h, g.stride_h), TILE) * g.stride_h : ty;
        // channel tiles per wavefront: as many as keep at least ~2 workgroups per compute unit
        int R = co_tiles >= 4 ? 4 : co_tiles >= 2 ? 2 : 1;
        while (R > 1 && (int64_t)gtx * gty * g.batch * ceil_div(co_tiles, R) < 512) R >>= 1;
        // steps a tile actually runs: a transposed convolution uses (K / stride)^2 taps per phase
        const int tile_steps = transposed ? ceil_div(g.kernel_h, g.stride_h) * ceil_div(g.kernel_w, g.stride_w) * (ci_p / 32) : steps;
        const bool ksplit = tile_steps >= 8;
        const int co_blocks = ceil_div(co_tiles, R);
        dim3 grid(gtx, gty, g.batch * co_blocks);
        note_kernel("conv_mfma_kernel");
#define DC_MFMA_L(TRF, KWV, RV, SV) conv_mfma_kernel<E16, TRF, KWV, RV, SV><<<grid, KWV * WAVE, 0, s>>>(p, (const E16 *)in, (const E16 *)packed, (const E16 *)bias, (E16 *)out, mask, out_mask, co_blocks, ci_p)
#define DC_MFMA(TRF)                                                                   \
    do {                                                                               \
        if (ksplit) {                                                                  \
            if (R == 4) DC_MFMA_L(TRF, 4, 4, 2);                                       \
            else if (R == 2) DC_MFMA_L(TRF, 4, 2, 2);                                  \
            else DC_MFMA_L(TRF, 4, 1, 4);                                              \
        } else {                                                                       \
            if (R == 4) DC_MFMA_L(TRF, 1, 4, 2);                                       \
            else if (R == 2) DC_MFMA_L(TRF, 1, 2, 2);                                  \
            else DC_MFMA_L(TRF, 1, 1, 4);                                              \
        }                                                                              \
    } while (0)
        if (transposed) DC_MFMA(true); else DC_MFMA(false);
#undef DC_MFMA
#undef DC_MFMA_L
    } else {
        dim3 grid(tx, ty, g.batch);
        note_kernel("conv_direct_kernel");
        int COT = pow2_ceil(g.out_c);
        if (COT > 256) COT = 256;
        if (dtype == DC_F32) {
            if (transposed)
                conv_direct_kernel<float, true><<<grid, 256, 0, s>>>(p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, COT);
            else
                conv_direct_kernel<float, false><<<grid, 256, 0, s>>>(p, (const float *)in, (const float *)filter, (const float *)bias, (float *)out, mask, out_mask, COT);
        } else if (dtype == DC_BF16) {
            if (transposed)
                conv_direct_kernel<bf16_t, true><<<grid, 256, 0, s>>>(p, (const bf16_t *)in, (const bf16_t *)filter, (const bf16_t *)bias, (bf16_t *)out, mask, out_mask, COT);
            else
                conv_direct_kernel<bf16_t, false><<<grid, 256, 0, s>>>(p, (const bf16_t *)in, (const bf16_t *)filter, (const bf16_t *)bias, (bf16_t *)out, mask, out_mask, COT);
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
}  // namespace

bool depthwise_closing_eligible(const dc_geometry &g, const ActEpilogue *epi, int dtype) {
    const ConvP p = make_params(g, dtype);
    const OpenAct none{};
    if (dtype == DC_F16)
        return try_depthwise_closing<half_t>(g, p, nullptr, nullptr, nullptr, nullptr, nullptr, epi, none, false, nullptr);
    if (dtype == DC_BF16)
        return try_depthwise_closing<bf16_t>(g, p, nullptr, nullptr, nullptr, nullptr, nullptr, epi, none, false, nullptr);
    return false;
}

hipError_t launch_depthwise_closing(const dc_geometry &g, const void *in, const void *filter, void *out,
                                    const int32_t *mask, int32_t *out_mask, const ActEpilogue *epi,
                                    const OpenAct &open, int dtype, hipStream_t s) {
    const ConvP p = make_params(g, dtype);
    const bool ok = dtype == DC_BF16
        ? try_depthwise_closing<bf16_t>(g, p, (const bf16_t *)in, (const bf16_t *)filter, (bf16_t *)out, mask, out_mask, epi, open, true, s)
        : try_depthwise_closing<half_t>(g, p, (const half_t *)in, (const half_t *)filter, (half_t *)out, mask, out_mask, epi, open, true, s);
    return ok ? hipGetLastError() : hipErrorInvalidValue;
}

hipError_t launch_conv(const dc_geometry &g, const void *in, const void *filter,
                       const void *packed, const void *bias, void *out, const int32_t *mask,
                       int32_t *out_mask, int dtype, bool transposed, const ActEpilogue *epi,
                       hipStream_t s) {
    if (dtype == DC_BF16)
        return launch_conv_t<bf16_t>(g, in, filter, packed, bias, out, mask, out_mask, dtype, transposed, epi, s);
    return launch_conv_t<half_t>(g, in, filter, packed, bias, out, mask, out_mask, dtype, transposed, epi, s);
}

}  // namespace dc
