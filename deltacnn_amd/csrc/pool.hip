// Delta pooling.
//   max: out = max_w(prev + M*delta) - max_w(prev) over in-bounds window pixels
//   avg: out = sum_w M*delta / (Kh*Kw)
// Arithmetic is fp32 for both tensor types with one rounding on store.
//
// pool_pixel_kernel   2x2 / 3x3 windows on small and mid-size maps: a lane group per output
//                     pixel, everything requested at once
// pool_scan_kernel    2x2 / 3x3 windows on very large maps: mask scan and compaction per wavefront
// pool_window_kernel  8x8 output tile per workgroup, mask dilation + compaction as for the
//                     convolutions; each compacted pixel is then handled by a group of G lanes
//                     that run along the channels with 16-byte vectors
// pool_global_kernel  1x1 output (float32 [B][C]); every workgroup owns a slice of channels
//                     and walks all input pixels, so the sum has a fixed order and needs no
//                     atomics
#include <type_traits>

#include "tile.hpp"

namespace dc {
namespace {

struct PoolQ {          // the literal zero that joins the maximum for bottom / right padding
    int zero_bottom;    // rows >= Hi inside the bottom padding when pad_top != pad_bottom
    int zero_right;     // columns >= Wi inside the right padding when pad_left != pad_right
    int pb, pr;
};

// K = 2, 3: square window of that size -- mask words, deltas and cached inputs of all taps are
// requested together from clamped addresses and selected afterwards (one memory round trip per
// output instead of one per tap); K = 0: any window, tap by tap.  Same order of operations.
template <typename T, int N, bool MAX, int K>
__global__ void __launch_bounds__(256)
pool_window_kernel(ConvP p, PoolQ q, const T *__restrict__ in, const T *__restrict__ prev,
                   T *__restrict__ out, const int32_t *__restrict__ mask,
                   int32_t *__restrict__ out_mask, int G) {
    __shared__ int s_list[TILE_PX];
    __shared__ int s_n;
    const int b = blockIdx.z;
    const int n = tile_mask_phase<false>(p, mask, out_mask, b, blockIdx.y * TILE,
                                         blockIdx.x * TILE, true, s_list, &s_n);
    if (n == 0) return;
    const int C = p.Ci;
    const int grp = threadIdx.x / G, gl = threadIdx.x & (G - 1), groups = 256 / G;
    const T *inb = in + (size_t)b * p.Hi * p.Wi * C;
    const T *pvb = MAX ? prev + (size_t)b * p.Hi * p.Wi * C : nullptr;
    const int32_t *mb = mask + (size_t)b * p.Hi * p.Wi;
    for (int idx = grp; idx < n; idx += groups) {
        const int code = s_list[idx];
        const int oy = code >> 16, ox = code & 0xffff;
        for (int c = gl * N; c < C; c += G * N) {
            float hi[N], hp[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                hi[j] = MAX ? -INFINITY : 0.f;
                hp[j] = -INFINITY;
            }
            constexpr int KK = K > 0 ? K * K : 1, KD = K > 0 ? K : 1;
            Vec<T, N> pd[KK], pp[KK];
            int pm[KK];
            if (K > 0) {
#pragma unroll
                for (int t = 0; t < KK; ++t) {
                    const int iy = min(max(oy * p.sh - p.pt + (t / KD) * p.dh, 0), p.Hi - 1);
                    const int ix = min(max(ox * p.sw - p.pl + (t % KD) * p.dw, 0), p.Wi - 1);
                    const int ip = iy * p.Wi + ix;
                    pm[t] = mb[ip];
                    pd[t] = vload<T, N>(inb + (size_t)ip * C + c);
                    if (MAX) pp[t] = vload<T, N>(pvb + (size_t)ip * C + c);
                }
            }
            for (int ky = 0; ky < (K > 0 ? K : p.Kh); ++ky) {  // constant trip counts unroll fully
                const int iy = oy * p.sh - p.pt + ky * p.dh;
                if (iy < 0) continue;
                if (iy >= p.Hi) {
                    if (MAX && q.zero_bottom && iy < p.Hi + q.pb) {
#pragma unroll
                        for (int j = 0; j < N; ++j) {
                            hi[j] = fmaxf(hi[j], 0.f);
                            hp[j] = fmaxf(hp[j], 0.f);
                        }
                    }
                    continue;
                }
                for (int kx = 0; kx < (K > 0 ? K : p.Kw); ++kx) {
                    const int ix = ox * p.sw - p.pl + kx * p.dw;
                    if (ix < 0) continue;
                    if (ix >= p.Wi) {
                        if (MAX && q.zero_right && ix < p.Wi + q.pr) {
#pragma unroll
                            for (int j = 0; j < N; ++j) {
                                hi[j] = fmaxf(hi[j], 0.f);
                                hp[j] = fmaxf(hp[j], 0.f);
                            }
                        }
                        continue;
                    }
                    const int ip = iy * p.Wi + ix;
                    const int t = K > 0 ? ky * K + kx : 0;
                    const bool act = (K > 0 ? pm[t] : mb[ip]) != 0;
                    if (!MAX && !act) continue;
                    Vec<T, N> d;
#pragma unroll
                    for (int j = 0; j < N; ++j) d.v[j] = T(0);
                    if (act) d = K > 0 ? pd[t] : vload<T, N>(inb + (size_t)ip * C + c);
                    if (MAX) {
                        Vec<T, N> pv = K > 0 ? pp[t] : vload<T, N>(pvb + (size_t)ip * C + c);
#pragma unroll
                        for (int j = 0; j < N; ++j) {
                            float pf = float(pv.v[j]);
                            hi[j] = fmaxf(hi[j], float(d.v[j]) + pf);
                            hp[j] = fmaxf(hp[j], pf);
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < N; ++j) hi[j] += float(d.v[j]);
                    }
                }
            }
            Vec<T, N> r;
            const float area = float(p.Kh * p.Kw);
#pragma unroll
            for (int j = 0; j < N; ++j) r.v[j] = MAX ? T(hi[j] - hp[j]) : T(hi[j] / area);
            vstore<T, N>(out + (((size_t)b * p.Ho + oy) * p.Wo + ox) * C + c, r);
        }
    }
}

// The K x K window kernel for maps of at least 2^18 outputs: a wavefront owns 64 consecutive
// output pixels, one per lane while the window's mask words are read and the output mask is
// written; the updated outputs are listed in LDS -- pixel, coordinates and the set of updated
// taps -- and served U at a time per lane group (one 16-byte vector per lane).  No workgroup
// barrier, a sparse map costs no idle groups, and the delta of a tap that was not updated is
// not fetched (its request goes to an updated tap's row, which is being read anyway).  Same
// operations in the same order as pool_window_kernel.
template <typename T, int N, bool MAX, int K>
__global__ void __launch_bounds__(256)
pool_scan_kernel(ConvP p, PoolQ q, const T *__restrict__ in, const T *__restrict__ prev,
                 T *__restrict__ out, const int32_t *__restrict__ mask,
                 int32_t *__restrict__ out_mask, int lg) {
    constexpr int KK = K * K;
    __shared__ int s_pix[4][WAVE], s_yx[4][WAVE], s_img[4][WAVE], s_taps[4][WAVE];
    const int Po = p.B * p.Ho * p.Wo, C = p.Ci;
    const int wave = wave_id(), lane = lane_id();
    const int po = (blockIdx.x * 4 + wave) * WAVE + lane;
    int taps = 0;  // bit t: tap t is inside the map and updated
    int yx, img;
    {
        const int pc = min(po, Po - 1);
        const int row = pc / p.Wo, ox = pc - row * p.Wo;
        const int b = row / p.Ho, oy = row - b * p.Ho;
        yx = (oy << 16) | ox;
        img = b * p.Hi * p.Wi;
        int mw[KK];
        bool inside[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const int iy = oy * p.sh - p.pt + (t / K) * p.dh, ix = ox * p.sw - p.pl + (t % K) * p.dw;
            inside[t] = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
            mw[t] = mask[(size_t)img + min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1)];
        }
#pragma unroll
        for (int t = 0; t < KK; ++t) taps |= (inside[t] && mw[t] != 0) ? 1 << t : 0;
    }
    if (po >= Po) taps = 0;
    if (po < Po) out_mask[po] = taps != 0 ? 1 : 0;
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
    constexpr int U = K == 2 ? 2 : 1;
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> pd[U][KK], pp[U][KK];
        bool valid[U];
        int pix[U], oy[U], ox[U], tp[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp, e = min(idx, n - 1);
            valid[u] = idx < n && mine;
            pix[u] = s_pix[wave][e];
            oy[u] = s_yx[wave][e] >> 16;
            ox[u] = s_yx[wave][e] & 0xffff;
            tp[u] = s_taps[wave][e];
            const size_t base = (size_t)s_img[wave][e];
            const int first = __builtin_ctz(tp[u]);  // an updated tap: the list holds no other pixels
            size_t ip[KK];
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                const int iy = min(max(oy[u] * p.sh - p.pt + (t / K) * p.dh, 0), p.Hi - 1);
                const int ix = min(max(ox[u] * p.sw - p.pl + (t % K) * p.dw, 0), p.Wi - 1);
                ip[t] = base + (size_t)iy * p.Wi + ix;
            }
            size_t ifirst = ip[0];
#pragma unroll
            for (int t = 1; t < KK; ++t) ifirst = first == t ? ip[t] : ifirst;
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                pd[u][t] = vload<T, N>(in + (((tp[u] >> t) & 1) ? ip[t] : ifirst) * C + c);
                if (MAX) pp[u][t] = vload<T, N>(prev + ip[t] * C + c);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
            float hi[N], hp[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                hi[j] = MAX ? -INFINITY : 0.f;
                hp[j] = -INFINITY;
            }
#pragma unroll
            for (int ky = 0; ky < K; ++ky) {
                const int iy = oy[u] * p.sh - p.pt + ky * p.dh;
                if (iy < 0) continue;
                if (iy >= p.Hi) {
                    if (MAX && q.zero_bottom && iy < p.Hi + q.pb) {
#pragma unroll
                        for (int j = 0; j < N; ++j) {
                            hi[j] = fmaxf(hi[j], 0.f);
                            hp[j] = fmaxf(hp[j], 0.f);
                        }
                    }
                    continue;
                }
#pragma unroll
                for (int kx = 0; kx < K; ++kx) {
                    const int ix = ox[u] * p.sw - p.pl + kx * p.dw;
                    if (ix < 0) continue;
                    if (ix >= p.Wi) {
                        if (MAX && q.zero_right && ix < p.Wi + q.pr) {
#pragma unroll
                            for (int j = 0; j < N; ++j) {
                                hi[j] = fmaxf(hi[j], 0.f);
                                hp[j] = fmaxf(hp[j], 0.f);
                            }
                        }
                        continue;
                    }
                    const int t = ky * K + kx;
                    const bool act = (tp[u] >> t) & 1;
                    if (!MAX && !act) continue;
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        const float d = act ? float(pd[u][t].v[j]) : 0.f;
                        if (MAX) {
                            const float pf = float(pp[u][t].v[j]);
                            hi[j] = fmaxf(hi[j], d + pf);
                            hp[j] = fmaxf(hp[j], pf);
                        } else {
                            hi[j] += d;
                        }
                    }
                }
            }
            Vec<T, N> r;
            const float area = float(K * K);
#pragma unroll
            for (int j = 0; j < N; ++j) r.v[j] = MAX ? T(hi[j] - hp[j]) : T(hi[j] / area);
            vstore<T, N>(out + (size_t)pix[u] * C + c, r);
        }
    }
}

// The K x K window kernel for maps that give pool_window_kernel too few tiles to fill the chip:
// one group of G lanes per OUTPUT pixel; every lane requests the window's mask words, the deltas
// and (for the maximum) the cached inputs of all taps at once from clamped addresses and selects
// afterwards -- one memory round trip, no workgroup barrier, no serial walk over a tile's pixels.
// Same operations in the same order as pool_window_kernel.
// UPD (maximum, windows that tile the map exactly: window == stride, no padding, no dilation): the
// cached input follows the input in the same launch -- prev += delta on the window's updated
// pixels, each of which belongs to this group's window alone -- what dc_add_to_dense does behind
// dc_pool otherwise.
template <typename T, int N, bool MAX, int K, bool UPD = false>
__global__ void __launch_bounds__(256)
pool_pixel_kernel(ConvP p, PoolQ q, const T *__restrict__ in, typename std::conditional<UPD, T, const T>::type *prev,
                  T *__restrict__ out, const int32_t *__restrict__ mask,
                  int32_t *__restrict__ out_mask, int lg) {
    constexpr int KK = K * K;
    const int Po = p.B * p.Ho * p.Wo, C = p.Ci;
    const int G = 1 << lg;
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int po = gid >> lg, gl = gid & (G - 1);
    if (po >= Po) return;
    const int row = po / p.Wo, ox = po - row * p.Wo;
    const int b = row / p.Ho, oy = row - b * p.Ho;
    const size_t base = (size_t)b * p.Hi * p.Wi;
    size_t ip[KK];
    int mw[KK];
    bool inside[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        const int iy = oy * p.sh - p.pt + (t / K) * p.dh, ix = ox * p.sw - p.pl + (t % K) * p.dw;
        inside[t] = iy >= 0 && iy < p.Hi && ix >= 0 && ix < p.Wi;
        ip[t] = base + (size_t)min(max(iy, 0), p.Hi - 1) * p.Wi + min(max(ix, 0), p.Wi - 1);
        mw[t] = mask[ip[t]];
    }
    for (int c0 = gl * N; c0 < C; c0 += G * N) {  // one pass unless C > 64 vectors
        Vec<T, N> pd[KK], pp[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            pd[t] = vload<T, N>(in + ip[t] * C + c0);
            if (MAX) pp[t] = vload<T, N>(prev + ip[t] * C + c0);
        }
        int taps = 0;
#pragma unroll
        for (int t = 0; t < KK; ++t) taps |= (inside[t] && mw[t] != 0) ? 1 << t : 0;
        if (c0 == gl * N && gl == 0) out_mask[po] = taps != 0 ? 1 : 0;
        if (taps == 0) return;  // the same for every lane of the group
        float hi[N], hp[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            hi[j] = MAX ? -INFINITY : 0.f;
            hp[j] = -INFINITY;
        }
#pragma unroll
        for (int ky = 0; ky < K; ++ky) {
            const int iy = oy * p.sh - p.pt + ky * p.dh;
            if (iy < 0) continue;
            if (iy >= p.Hi) {
                if (MAX && q.zero_bottom && iy < p.Hi + q.pb) {
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        hi[j] = fmaxf(hi[j], 0.f);
                        hp[j] = fmaxf(hp[j], 0.f);
                    }
                }
                continue;
            }
#pragma unroll
            for (int kx = 0; kx < K; ++kx) {
                const int ix = ox * p.sw - p.pl + kx * p.dw;
                if (ix < 0) continue;
                if (ix >= p.Wi) {
                    if (MAX && q.zero_right && ix < p.Wi + q.pr) {
#pragma unroll
                        for (int j = 0; j < N; ++j) {
                            hi[j] = fmaxf(hi[j], 0.f);
                            hp[j] = fmaxf(hp[j], 0.f);
                        }
                    }
                    continue;
                }
                const int t = ky * K + kx;
                const bool act = (taps >> t) & 1;
                if (!MAX && !act) continue;
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    const float d = act ? float(pd[t].v[j]) : 0.f;
                    if (MAX) {
                        const float pf = float(pp[t].v[j]);
                        hi[j] = fmaxf(hi[j], d + pf);
                        hp[j] = fmaxf(hp[j], pf);
                    } else {
                        hi[j] += d;
                    }
                }
            }
        }
        Vec<T, N> r;
        const float area = float(K * K);
#pragma unroll
        for (int j = 0; j < N; ++j) r.v[j] = MAX ? T(hi[j] - hp[j]) : T(hi[j] / area);
        vstore<T, N>(out + (size_t)po * C + c0, r);
        if (UPD) {
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                if (!((taps >> t) & 1)) continue;
                Vec<T, N> nv;
#pragma unroll
                for (int j = 0; j < N; ++j) nv.v[j] = pp[t].v[j] + pd[t].v[j];
                vstore<T, N>(const_cast<T *>(prev) + ip[t] * C + c0, nv);  // UPD: prev is not const
            }
        }
    }
}

// 1x1 output: grid (channel slices, batch); a workgroup's 4 wavefronts stride over the window
// taps, each lane owns one channel, partial results meet in LDS.
template <typename T, bool MAX>
__global__ void __launch_bounds__(256)
pool_global_kernel(ConvP p, PoolQ q, const T *__restrict__ in, const T *__restrict__ prev,
                   float *__restrict__ out, const int32_t *__restrict__ mask,
                   int32_t *__restrict__ out_mask) {
    __shared__ float s_hi[4][WAVE], s_hp[4][WAVE];
    __shared__ int s_any[4];
    const int b = blockIdx.y;
    const int C = p.Ci;
    const int c = blockIdx.x * WAVE + lane_id();
    const int wave = threadIdx.x / WAVE;
    const int npx = p.Hi * p.Wi;
    const int K2 = p.Kh * p.Kw;
    const T *inb = in + (size_t)b * npx * C;
    const T *pvb = MAX ? prev + (size_t)b * npx * C : nullptr;
    const int32_t *mb = mask + (size_t)b * npx;
    float hi = MAX ? -INFINITY : 0.f, hp = -INFINITY;
    int any = 0;
    for (int tap = wave; tap < K2; tap += 4) {
        const int ky = tap / p.Kw, kx = tap - ky * p.Kw;
        const int iy = ky * p.dh - p.pt, ix = kx * p.dw - p.pl;
        if (iy < 0 || ix < 0) continue;
        if (iy >= p.Hi || ix >= p.Wi) {
            const bool zero = iy >= p.Hi ? (q.zero_bottom && iy < p.Hi + q.pb)
                                         : (q.zero_right && ix < p.Wi + q.pr);
            if (MAX && zero) {
                hi = fmaxf(hi, 0.f);
                hp = fmaxf(hp, 0.f);
            }
            continue;
        }
        const int ip = iy * p.Wi + ix;
        const bool act = mb[ip] != 0;  // wave-uniform
        any |= act ? 1 : 0;
        if (c >= C) continue;
        if (MAX) {
            float pf = float(pvb[(size_t)ip * C + c]);
            float d = act ? float(inb[(size_t)ip * C + c]) : 0.f;
            hi = fmaxf(hi, d + pf);
            hp = fmaxf(hp, pf);
        } else if (act) {
            hi += float(inb[(size_t)ip * C + c]);
        }
    }
    s_hi[wave][lane_id()] = hi;
    s_hp[wave][lane_id()] = hp;
    if (lane_id() == 0) s_any[wave] = any;
    __syncthreads();
    if (wave == 0) {
        for (int w = 1; w < 4; ++w) {
            if (MAX) {
                hi = fmaxf(hi, s_hi[w][lane_id()]);
                hp = fmaxf(hp, s_hp[w][lane_id()]);
            } else {
                hi += s_hi[w][lane_id()];
            }
            any |= s_any[w];
        }
        if (c < C) out[(size_t)b * C + c] = any ? (MAX ? hi - hp : hi / float(K2)) : 0.f;
        if (blockIdx.x == 0 && lane_id() == 0 && out_mask != nullptr) out_mask[b] = any;
    }
}

// 1x1 output over the whole unpadded map (global pooling), channels in 16-byte vectors:
// a workgroup owns VPB channel vectors and splits the pixels over 256 / VPB slices; every
// load is unconditional (the mask word selects afterwards), partial results meet in LDS and
// are combined slice by slice in ascending order, so the sum has a fixed order and needs no
// atomics.  OutT is float (the reference's accumulator protocol) or T (cast fused).
// DENS (average, OutT == T): the DCDensify that follows a network's global pooling runs on the
// pooled delta as it leaves the reduction -- acc += delta if any pixel of the map was updated,
// dense = acc -- with the pooled delta rounded to T first, as the separate launches have it;
// the delta itself and its one-pixel mask are not stored.
template <typename T, typename OutT, bool MAX, bool DENS = false>
__global__ void __launch_bounds__(256)
pool_global_vec_kernel(int npx, int C, const T *__restrict__ in, const T *__restrict__ prev,
                       OutT *__restrict__ out, const int32_t *__restrict__ mask,
                       int32_t *__restrict__ out_mask, T *__restrict__ acc = nullptr,
                       T *__restrict__ dense = nullptr) {
    constexpr int N = Vec16<T>::N, VPB = 8, SL = 256 / VPB;
    __shared__ float s_hi[SL][VPB * N], s_hp[MAX ? SL : 1][VPB * N];
    const int b = blockIdx.y;
    T held = T(0);  // the accumulated value of this thread's channel, requested with the map
    if (DENS && threadIdx.x < VPB * N && blockIdx.x * VPB * N + threadIdx.x < C)
        held = acc[(size_t)b * C + blockIdx.x * VPB * N + threadIdx.x];
    const int vl = threadIdx.x % VPB, sl = threadIdx.x / VPB;
    const int c = (blockIdx.x * VPB + vl) * N;
    const int cc = min(c, C - N);
    const T *inb = in + (size_t)b * npx * C;
    const T *pvb = MAX ? prev + (size_t)b * npx * C : nullptr;
    const int32_t *mb = mask + (size_t)b * npx;
    float hi[N], hp[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
        hi[j] = MAX ? -INFINITY : 0.f;
        hp[j] = -INFINITY;
    }
    int any = 0;
    for (int ip = sl; ip < npx; ip += SL) {
        const int m = mb[ip];
        const Vec<T, N> d = vload<T, N>(inb + (size_t)ip * C + cc);
        Vec<T, N> pf;
        if (MAX) pf = vload<T, N>(pvb + (size_t)ip * C + cc);
        any |= m;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const float dv = m != 0 ? float(d.v[j]) : 0.f;
            if (MAX) {
                hi[j] = fmaxf(hi[j], dv + float(pf.v[j]));
                hp[j] = fmaxf(hp[j], float(pf.v[j]));
            } else {
                hi[j] += dv;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < N; ++j) {
        s_hi[sl][vl * N + j] = hi[j];
        if (MAX) s_hp[sl][vl * N + j] = hp[j];
    }
    const int wg_any = __syncthreads_or(any);
    if (threadIdx.x < VPB * N) {
        const int ch = blockIdx.x * VPB * N + threadIdx.x;
        float r = s_hi[0][threadIdx.x], rp = MAX ? s_hp[0][threadIdx.x] : 0.f;
        for (int s2 = 1; s2 < SL; ++s2) {
            if (MAX) {
                r = fmaxf(r, s_hi[s2][threadIdx.x]);
                rp = fmaxf(rp, s_hp[s2][threadIdx.x]);
            } else {
                r += s_hi[s2][threadIdx.x];
            }
        }
        if (ch < C) {
            const OutT pooled = OutT(wg_any ? (MAX ? r - rp : r / float(npx)) : 0.f);
            if (DENS) {
                if (wg_any) {
                    held = T(pooled) + held;
                    acc[(size_t)b * C + ch] = held;
                }
                dense[(size_t)b * C + ch] = held;
            } else {
                out[(size_t)b * C + ch] = pooled;
            }
        }
    }
    if (!DENS && blockIdx.x == 0 && threadIdx.x == 0 && out_mask != nullptr) out_mask[b] = wg_any ? 1 : 0;
}

template <typename T>
hipError_t pool_t(const dc_geometry &g, const T *in, const T *prev, void *out, const int32_t *mask,
                  int32_t *out_mask, int mode, bool out_f32, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    ConvP p;
    p.B = g.batch; p.Hi = g.in_h; p.Wi = g.in_w; p.Ci = g.in_c;
    p.Ho = g.out_h; p.Wo = g.out_w; p.Co = g.in_c;
    p.Kh = g.kernel_h; p.Kw = g.kernel_w; p.sh = g.stride_h; p.sw = g.stride_w;
    p.dh = g.dilation_h; p.dw = g.dilation_w; p.pt = g.pad_top; p.pl = g.pad_left;
    p.ci_g = p.co_g = 1; p.w_co = 0; p.swz = 0;
    PoolQ q;
    q.pb = g.pad_bottom; q.pr = g.pad_right;
    q.zero_bottom = g.pad_top != g.pad_bottom;
    q.zero_right = g.pad_left != g.pad_right;
    if (g.out_h == 1 && g.out_w == 1) {
        const bool whole = g.kernel_h == g.in_h && g.kernel_w == g.in_w && g.pad_top == 0 && g.pad_left == 0 &&
                           g.pad_bottom == 0 && g.pad_right == 0 && g.dilation_h == 1 && g.dilation_w == 1;
        if (whole && g.in_c % N == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)prev & 15) == 0) {
            note_kernel("pool_global_vec_kernel");
            dim3 vgrid(ceil_div(g.in_c / N, 8), g.batch);
            const int npx = g.in_h * g.in_w;
#define DC_PG(OT, MX) pool_global_vec_kernel<T, OT, MX><<<vgrid, 256, 0, s>>>(npx, g.in_c, in, prev, (OT *)out, mask, out_mask)
            if (mode == DC_POOL_MAX) {
                if (out_f32) DC_PG(float, true); else DC_PG(T, true);
            } else {
                if (out_f32) DC_PG(float, false); else DC_PG(T, false);
            }
#undef DC_PG
            return hipGetLastError();
        }
        if (!out_f32) return hipErrorInvalidValue;  // checked by the caller: cannot happen
        note_kernel("pool_global_kernel");
        dim3 grid(ceil_div(g.in_c, WAVE), g.batch);
        if (mode == DC_POOL_MAX)
            pool_global_kernel<T, true><<<grid, 256, 0, s>>>(p, q, in, prev, (float *)out, mask, out_mask);
        else
            pool_global_kernel<T, false><<<grid, 256, 0, s>>>(p, q, in, prev, (float *)out, mask, out_mask);
        return hipGetLastError();
    }
    dim3 grid(ceil_div(g.out_w, TILE), ceil_div(g.out_h, TILE), g.batch);
    const bool vec = g.in_c % N == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                     ((uintptr_t)prev & 15) == 0;
    int G = pow2_ceil(vec ? g.in_c / N : g.in_c);
    if (G > WAVE) G = WAVE;
    const int ksq = (g.kernel_h == g.kernel_w && (g.kernel_h == 2 || g.kernel_h == 3)) ? g.kernel_h : 0;
    const int64_t po = (int64_t)g.batch * g.out_h * g.out_w;
    if (ksq > 0 && vec && g.in_c / N <= WAVE && po >= (1 << 18) && po < (1ll << 31) && g.out_h < 65536 && g.out_w < 65536 &&
        (int64_t)g.batch * g.in_h * g.in_w < (1ll << 31)) {
        note_kernel("pool_scan_kernel");
        const dim3 sgrid((unsigned)ceil_div64(po, 4 * WAVE));
        int lg = 0;
        while ((1 << lg) < G) ++lg;
#define DC_PS(MX, KV) pool_scan_kernel<T, N, MX, KV><<<sgrid, 256, 0, s>>>(p, q, in, prev, (T *)out, mask, out_mask, lg)
        if (mode == DC_POOL_MAX) { if (ksq == 2) DC_PS(true, 2); else DC_PS(true, 3); }
        else { if (ksq == 2) DC_PS(false, 2); else DC_PS(false, 3); }
#undef DC_PS
        return hipGetLastError();
    }
    // small and mid-size maps: a lane group per output pixel, one memory round trip (measured
    // against the tile kernel, whose few workgroups walk their pixels one after the other)
    if (ksq > 0 && vec && po * G <= (1 << 20) && (int64_t)g.batch * g.in_h * g.in_w < (1ll << 31)) {
        note_kernel("pool_pixel_kernel");
        const int64_t lanes = po * G;
        const int block = lanes <= 2048 * WAVE ? WAVE : 256;
        const dim3 pgrid((unsigned)ceil_div64(lanes, block));
        int lg = 0;
        while ((1 << lg) < G) ++lg;
#define DC_PP(MX, KV) pool_pixel_kernel<T, N, MX, KV><<<pgrid, block, 0, s>>>(p, q, in, prev, (T *)out, mask, out_mask, lg)
        if (mode == DC_POOL_MAX) { if (ksq == 2) DC_PP(true, 2); else DC_PP(true, 3); }
        else { if (ksq == 2) DC_PP(false, 2); else DC_PP(false, 3); }
#undef DC_PP
        return hipGetLastError();
    }
    note_kernel("pool_window_kernel");
#define DC_POOL(NN, MX)                                                                                           \
    do {                                                                                                          \
        if (ksq == 2) pool_window_kernel<T, NN, MX, 2><<<grid, 256, 0, s>>>(p, q, in, prev, (T *)out, mask, out_mask, G); \
        else if (ksq == 3) pool_window_kernel<T, NN, MX, 3><<<grid, 256, 0, s>>>(p, q, in, prev, (T *)out, mask, out_mask, G); \
        else pool_window_kernel<T, NN, MX, 0><<<grid, 256, 0, s>>>(p, q, in, prev, (T *)out, mask, out_mask, G);   \
    } while (0)
    if (mode == DC_POOL_MAX) {
        if (vec) DC_POOL(N, true); else DC_POOL(1, true);
    } else {
        if (vec) DC_POOL(N, false); else DC_POOL(1, false);
    }
#undef DC_POOL
    return hipGetLastError();
}

}  // namespace

// dc_pool_update: maximum pooling whose windows tile the map exactly, on a map of the per-pixel
// kernel's range, channels in whole 16-byte vectors.
bool pool_update_eligible(const dc_geometry &g, const void *in, const void *prev, const void *out, int dtype) {
    const int n = dtype == DC_F32 ? 4 : 8;
    const bool sq = g.kernel_h == g.kernel_w && (g.kernel_h == 2 || g.kernel_h == 3);
    const bool tiles = g.stride_h == g.kernel_h && g.stride_w == g.kernel_w && g.dilation_h == 1 && g.dilation_w == 1 &&
                       g.pad_top == 0 && g.pad_left == 0 && g.pad_bottom == 0 && g.pad_right == 0 &&
                       g.in_h == g.out_h * g.stride_h && g.in_w == g.out_w * g.stride_w;
    const bool vec = g.in_c % n == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)prev & 15) == 0;
    int G = pow2_ceil(g.in_c / std::max(n, 1));
    if (G > WAVE) G = WAVE;
    const int64_t po = (int64_t)g.batch * g.out_h * g.out_w;
    return sq && tiles && vec && g.in_c / n <= WAVE && po * G <= (1 << 20) && (int64_t)g.batch * g.in_h * g.in_w < (1ll << 31);
}

namespace {
template <typename T>
hipError_t pool_update_t(const dc_geometry &g, const T *in, T *prev, T *out, const int32_t *mask, int32_t *out_mask,
                         hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    ConvP p;
    p.B = g.batch; p.Hi = g.in_h; p.Wi = g.in_w; p.Ci = g.in_c;
    p.Ho = g.out_h; p.Wo = g.out_w; p.Co = g.in_c;
    p.Kh = g.kernel_h; p.Kw = g.kernel_w; p.sh = g.stride_h; p.sw = g.stride_w;
    p.dh = p.dw = 1; p.pt = p.pl = 0;
    p.ci_g = p.co_g = 1; p.w_co = 0; p.swz = 0;
    PoolQ q;
    q.pb = q.pr = 0;
    q.zero_bottom = q.zero_right = false;
    int G = pow2_ceil(g.in_c / N);
    if (G > WAVE) G = WAVE;
    const int64_t lanes = (int64_t)g.batch * g.out_h * g.out_w * G;
    const int block = lanes <= 2048 * WAVE ? WAVE : 256;
    const dim3 pgrid((unsigned)ceil_div64(lanes, block));
    int lg = 0;
    while ((1 << lg) < G) ++lg;
    note_kernel("pool_pixel_kernel");
    if (g.kernel_h == 2) pool_pixel_kernel<T, N, true, 2, true><<<pgrid, block, 0, s>>>(p, q, in, prev, out, mask, out_mask, lg);
    else pool_pixel_kernel<T, N, true, 3, true><<<pgrid, block, 0, s>>>(p, q, in, prev, out, mask, out_mask, lg);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_pool_update(const dc_geometry &g, const void *in, void *prev, void *out, const int32_t *mask,
                              int32_t *out_mask, int dtype, hipStream_t s) {
    if (dtype == DC_F32) return pool_update_t<float>(g, (const float *)in, (float *)prev, (float *)out, mask, out_mask, s);
    if (dtype == DC_BF16) return pool_update_t<bf16_t>(g, (const bf16_t *)in, (bf16_t *)prev, (bf16_t *)out, mask, out_mask, s);
    return pool_update_t<half_t>(g, (const half_t *)in, (half_t *)prev, (half_t *)out, mask, out_mask, s);
}

bool pool_global_casts(const dc_geometry &g, const void *in, const void *prev, int dtype) {
    const int n = dtype == DC_F32 ? 4 : 8;
    return g.out_h == 1 && g.out_w == 1 && g.kernel_h == g.in_h && g.kernel_w == g.in_w && g.pad_top == 0 &&
           g.pad_left == 0 && g.pad_bottom == 0 && g.pad_right == 0 && g.dilation_h == 1 &&
           g.dilation_w == 1 && g.in_c % n == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)prev & 15) == 0;
}

namespace {
template <typename T>
hipError_t pool_densify_t(const dc_geometry &g, const T *in, const int32_t *mask, T *acc, T *dense,
                          hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    note_kernel("pool_global_vec_kernel");
    dim3 vgrid(ceil_div(g.in_c / N, 8), g.batch);
    pool_global_vec_kernel<T, T, false, true><<<vgrid, 256, 0, s>>>(g.in_h * g.in_w, g.in_c, in, nullptr, nullptr, mask,
                                                                    nullptr, acc, dense);
    return hipGetLastError();
}
}  // namespace

// Global average pooling + DCDensify in one launch; the caller has checked pool_global_casts.
hipError_t launch_pool_densify(const dc_geometry &g, const void *in, const int32_t *mask, void *acc,
                               void *dense, int dtype, hipStream_t s) {
    if (dtype == DC_F32) return pool_densify_t<float>(g, (const float *)in, mask, (float *)acc, (float *)dense, s);
    if (dtype == DC_BF16) return pool_densify_t<bf16_t>(g, (const bf16_t *)in, mask, (bf16_t *)acc, (bf16_t *)dense, s);
    return pool_densify_t<half_t>(g, (const half_t *)in, mask, (half_t *)acc, (half_t *)dense, s);
}

hipError_t launch_pool(const dc_geometry &g, const void *in, const void *prev, void *out,
                       const int32_t *mask, int32_t *out_mask, int mode, int dtype, bool out_f32,
                       hipStream_t s) {
    if (dtype == DC_F32)
        return pool_t<float>(g, (const float *)in, (const float *)prev, out, mask, out_mask, mode, true, s);
    if (dtype == DC_BF16)
        return pool_t<bf16_t>(g, (const bf16_t *)in, (const bf16_t *)prev, out, mask, out_mask, mode, out_f32, s);
    return pool_t<half_t>(g, (const half_t *)in, (const half_t *)prev, out, mask, out_mask, mode, out_f32, s);
}

}  // namespace dc
