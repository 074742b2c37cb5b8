// Activation + truncation of one pixel held in registers by a group of G lanes.
//
//   T = trunc + delta;  S = T + prev;  D = act(S) - act(prev)
//   keep  (max: any |D| > thr; norm: sqrt(sum D^2) > thr; rms: sqrt(sum D^2 / C) > thr):
//         prev = S, delta = D, trunc = 0
//   else: trunc = T, the mask word is cleared (delta is left as it is)
//
// Used by the stand-alone activation kernel and as the epilogue of the depthwise
// convolution.  Every operation rounds on its own in the tensor's type (compile with
// -ffp-contract=off), so the keep/drop decision is reproducible bit for bit.
#pragma once

#include "common.hpp"

namespace dc {

__device__ __forceinline__ float group_sum(float v, int G) {
    for (int o = 1; o < G; o <<= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// `dl[it]` holds channels (it*G + gl)*N .. +N of the incoming delta for pixel `p`, `q` / `tr`
// the same channels of the cached pre-activation and of the truncated remainder (loaded by the
// caller as early as it can, see load_state; only meaningful where `valid` and the channel
// offset is < C).  All lanes of the wavefront must call this (it contains wave-wide ballots);
// with G > 64 (one pixel per workgroup, mode max only) all wavefronts of the workgroup must.
// Returns whether the pixel was kept.
template <typename T, int ITERS>
__device__ __forceinline__ void load_state(Vec<T, Vec16<T>::N> (&q)[ITERS],
                                           Vec<T, Vec16<T>::N> (&tr)[ITERS], bool valid, size_t p,
                                           int gl, int G, int C, const T *__restrict__ prev,
                                           const T *__restrict__ trunc) {
    constexpr int N = Vec16<T>::N;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int c = (it * G + gl) * N;
        if (valid && c < C) {
            q[it] = vload<T, N>(prev + p * C + c);
            tr[it] = vload<T, N>(trunc + p * C + c);
        }
    }
}

template <typename T, int ITERS, int ACT>
__device__ __forceinline__ bool act_trunc_pixel(Vec<T, Vec16<T>::N> (&dl)[ITERS],
                                                const Vec<T, Vec16<T>::N> (&q)[ITERS],
                                                const Vec<T, Vec16<T>::N> (&tr)[ITERS], bool valid,
                                                size_t p, int gl, int G, int C,
                                                T *__restrict__ delta, T *__restrict__ prev,
                                                T *__restrict__ trunc, int32_t *__restrict__ mask,
                                                T thr, int mode) {
    constexpr int N = Vec16<T>::N;
    Vec<T, N> t[ITERS], s[ITERS];
    bool hit = false;
    float sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int c = (it * G + gl) * N;
        if (valid && c < C) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                t[it].v[j] = tr[it].v[j] + dl[it].v[j];
                s[it].v[j] = t[it].v[j] + q[it].v[j];
                const T d = act_apply<T>(s[it].v[j], ACT) - act_apply<T>(q[it].v[j], ACT);
                dl[it].v[j] = d;
                hit |= tabs(d) > thr;
            }
        }
    }
    if (mode != DC_TRUNC_MAX) {  // uniform: the squares are only needed by the norm modes
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = (it * G + gl) * N;
            if (valid && c < C) {
#pragma unroll
                for (int j = 0; j < N; ++j) sq += float(dl[it].v[j]) * float(dl[it].v[j]);
            }
        }
    }
    bool keep;
    if (mode == DC_TRUNC_MAX) {
        keep = group_any(hit, G);
        // a group wider than a wavefront is a whole workgroup working on one pixel
        if (G > WAVE) keep = __syncthreads_or(keep) != 0;
    } else {
        sq = group_sum(sq, G);
        if (mode == DC_TRUNC_RMS) sq /= float(C);
        keep = sqrtf(sq) > float(thr);
    }
    if (valid) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = (it * G + gl) * N;
            if (c < C) {
                const size_t off = p * C + c;
                if (keep) {
                    Vec<T, N> z;
#pragma unroll
                    for (int j = 0; j < N; ++j) z.v[j] = T(0);
                    vstore<T, N>(prev + off, s[it]);
                    vstore<T, N>(delta + off, dl[it]);
                    // (a remainder that is zero already -- the pixel was kept last time too -- is not stored again)
                    if (any_bits(tr[it])) vstore<T, N>(trunc + off, z);
                } else {
                    vstore<T, N>(trunc + off, t[it]);
                }
            }
        }
        if (!keep && gl == 0) mask[p] = 0;
    }
    return keep;
}

// One pixel per workgroup of 128 / 256 lanes, one vector per lane: for rows of more than 64
// vectors on small maps, where a lane holding several vectors makes the wavefront's
// instruction stream -- which is the kernel time at this size -- several times longer.
inline int wide_group(int nvec, int64_t pixels) {
    if (nvec <= WAVE || nvec > 256 || pixels > 1024) return 0;
    return nvec <= 128 ? 128 : 256;
}

// Lanes per pixel for `nvec` 16-byte vectors per row when a lane may hold up to `max_iters`.
inline int group_lanes(int nvec, int max_iters) {
    int g = pow2_ceil(ceil_div(nvec, max_iters));
    return g > WAVE ? WAVE : g;
}

// Small tensors favour parallelism (one vector per lane, some idle lanes); large ones favour
// lane efficiency (several vectors per lane).
inline int pick_group(int nvec, int64_t pixels, int max_iters) {
    const int wide = group_lanes(nvec, 1);
    if (pixels * wide <= (1 << 18) || nvec <= 1) return wide;
    int best = wide, best_waste = wide * ceil_div(nvec, wide) - nvec;
    for (int it = 2; it <= max_iters; ++it) {
        int g = group_lanes(nvec, it);
        int waste = g * ceil_div(nvec, g) - nvec;
        if (waste < best_waste) best = g, best_waste = waste;
    }
    return best;
}

inline int log2i(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

}  // namespace dc
