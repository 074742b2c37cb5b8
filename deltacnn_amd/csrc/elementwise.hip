// Bandwidth-bound per-pixel operators of the delta path: sparsify, activation + truncation,
// densify, add, add-to-dense, nearest upsample, concatenate, per-channel scale/offset.
//
// Common shape: features are NHWC, so a pixel is a contiguous row of C values.  A pixel is
// handled by an aligned group of G lanes (G a power of two, chosen on the host so that a
// group covers the row with 16-byte vectors); a wavefront therefore handles 64/G pixels and
// the grid has one group per pixel.  Groups of inactive pixels read their mask word and
// leave; per-pixel decisions are group-wide ballots.  One group per pixel (instead of a loop
// over pixels inside a wavefront) keeps small feature maps -- a 7x7 map is 49 pixels -- spread
// over many wavefronts, which is what matters at batch 1.
//
// Compiled with -ffp-contract=off: every arithmetic operation rounds on its own, in the
// tensor's own type, which is what makes masks reproducible bit for bit.
#include "epilogue.hpp"

namespace dc {
namespace {

// Pixel and lane-in-group of this thread for groups of G = 1 << lg lanes.
__device__ __forceinline__ void group_coords(int lg, int &p, int &gl) {
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    p = gid >> lg;
    gl = gid & ((1 << lg) - 1);
}

// ------------------------------------------------------------------------------- sparsify
// delta = in - prev; the pixel is active if any channel passes the compare (`ge`: >= instead
// of >, the fp16 even-C rule); active pixels write delta and prev := in for all channels.
template <typename T, int ITERS>
__global__ void __launch_bounds__(256)
sparsify_vec_kernel(const T *__restrict__ in, T *__restrict__ prev, T *__restrict__ delta,
                    int32_t *__restrict__ mask, float thr_f, int P, int C, int G, bool ge) {
    constexpr int N = Vec16<T>::N;
    const T thr = T(thr_f);
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int p = gid / G;
    const int gl = gid & (G - 1);
    const bool valid = p < P;
    Vec<T, N> x[ITERS], d[ITERS];
    bool hit = false;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        int c = (it * G + gl) * N;
        if (valid && c < C) {
            size_t off = (size_t)p * C + c;
            x[it] = vload<T, N>(in + off);
            Vec<T, N> q = vload<T, N>(prev + off);
#pragma unroll
            for (int j = 0; j < N; ++j) {
                d[it].v[j] = x[it].v[j] - q.v[j];
                T a = tabs(d[it].v[j]);
                hit |= ge ? !(a < thr) : (a > thr);
            }
        }
    }
    const bool any = group_any(hit, G);
    if (valid && any) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            int c = (it * G + gl) * N;
            if (c < C) {
                size_t off = (size_t)p * C + c;
                vstore<T, N>(delta + off, d[it]);
                vstore<T, N>(prev + off, x[it]);
            }
        }
    }
    if (valid && gl == 0) mask[p] = any ? 1 : 0;
}

// Any C / alignment: scalar, two passes (scan, then recompute and write).
template <typename T>
__global__ void __launch_bounds__(256)
sparsify_gen_kernel(const T *__restrict__ in, T *__restrict__ prev, T *__restrict__ delta,
                    int32_t *__restrict__ mask, float thr_f, int P, int C, int G, bool ge) {
    const T thr = T(thr_f);
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int p = gid / G;
    const int gl = gid & (G - 1);
    const bool valid = p < P;
    bool hit = false;
    if (valid) {
        for (int c = gl; c < C; c += G) {
            size_t off = (size_t)p * C + c;
            T a = tabs(T(in[off] - prev[off]));
            hit |= ge ? !(a < thr) : (a > thr);
        }
    }
    const bool any = group_any(hit, G);
    if (valid && any) {
        for (int c = gl; c < C; c += G) {
            size_t off = (size_t)p * C + c;
            T xi = in[off];
            delta[off] = xi - prev[off];
            prev[off] = xi;
        }
    }
    if (valid && gl == 0) mask[p] = any ? 1 : 0;
}

// ----------------------------------------------------------------- activation + truncation
// EAGER (small maps): delta, cached state and mask word are requested together -- their
// addresses depend on coordinates only -- so the kernel is one memory round trip; what is
// loaded for inactive pixels is dropped.
template <typename T, int ITERS, int ACT, bool EAGER>
__global__ void __launch_bounds__(256)
act_trunc_vec_kernel(T *__restrict__ delta, T *__restrict__ prev, T *__restrict__ trunc,
                     int32_t *__restrict__ mask, float thr_f, int mode, int P, int C, int lg) {
    constexpr int N = Vec16<T>::N;
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    Vec<T, N> dl[ITERS], q[ITERS], tr[ITERS];
    if (EAGER) {
        const size_t row = (size_t)min(p, P - 1) * C;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = min((it * G + gl) * N, C - N);
            dl[it] = vload<T, N>(delta + row + c);
            q[it] = vload<T, N>(prev + row + c);
            tr[it] = vload<T, N>(trunc + row + c);
        }
    }
    const bool valid = p < P && mask[min(p, P - 1)] != 0;
    if (ballot(valid) == 0) return;
    if (!EAGER) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int c = (it * G + gl) * N;
            if (valid && c < C) dl[it] = vload<T, N>(delta + (size_t)p * C + c);
        }
        load_state<T, ITERS>(q, tr, valid, (size_t)p, gl, G, C, prev, trunc);
    }
    act_trunc_pixel<T, ITERS, ACT>(dl, q, tr, valid, (size_t)p, gl, G, C, delta, prev, trunc, mask,
                                   T(thr_f), mode);
}

// The activation / truncation of several small tensors in one launch (the branches of a
// multi-resolution network): a workgroup looks up the tensor its number falls into and runs the
// eager form above on it.  Maximum norm only -- its keep decision does not depend on how the
// channels of a pixel are spread over lanes, so the results are those of the separate launches.
template <typename T>
struct ActItemD {
    T *delta, *prev, *trunc;
    int32_t *mask;
    float thr;
    int P, C, lg, iters, first;
};

template <typename T>
struct ActGroupD {
    int n;
    ActItemD<T> it[CONV_GROUP_MAX];
};

template <typename T, int ITERS, int ACT>
__device__ __forceinline__ void act_trunc_group_item(const ActItemD<T> &it, int gid) {
    constexpr int N = Vec16<T>::N;
    const int G = 1 << it.lg, P = it.P, C = it.C;
    const int p = gid >> it.lg, gl = gid & (G - 1);
    Vec<T, N> dl[ITERS], q[ITERS], tr[ITERS];
    const size_t row = (size_t)min(p, P - 1) * C;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
        const int c = min((i * G + gl) * N, C - N);
        dl[i] = vload<T, N>(it.delta + row + c);
        q[i] = vload<T, N>(it.prev + row + c);
        tr[i] = vload<T, N>(it.trunc + row + c);
    }
    const bool valid = p < P && it.mask[min(p, P - 1)] != 0;
    if (ballot(valid) == 0) return;
    act_trunc_pixel<T, ITERS, ACT>(dl, q, tr, valid, (size_t)p, gl, G, C, it.delta, it.prev, it.trunc, it.mask,
                                   T(it.thr), DC_TRUNC_MAX);
}

template <typename T, int ACT>
__global__ void __launch_bounds__(256)
act_trunc_group_kernel(ActGroupD<T> g) {
    int idx = 0;
#pragma unroll
    for (int i = 1; i < CONV_GROUP_MAX; ++i)
        if (i < g.n && (int)blockIdx.x >= g.it[i].first) idx = i;
    const ActItemD<T> &it = g.it[idx];
    const int gid = (blockIdx.x - it.first) * 256 + threadIdx.x;
    if (it.iters == 1) act_trunc_group_item<T, 1, ACT>(it, gid);
    else if (it.iters == 2) act_trunc_group_item<T, 2, ACT>(it, gid);
    else act_trunc_group_item<T, 4, ACT>(it, gid);
}

// Large maps: a wavefront scans the mask words of 64 consecutive pixels in one coalesced read,
// compacts the active ones by ballot and then works through them 64 / G pixels at a time.  With
// one group per pixel a sparse map costs a wavefront launch per 64 / G pixels, most of which
// leave at once; here a wavefront exists per 64 pixels and only active pixels occupy lanes.
constexpr int SCAN_MIN_PIXELS = 1 << 18;  // 4096 wavefronts: enough to fill the chip

template <typename T, int ACT>
__global__ void __launch_bounds__(256)
act_trunc_scan_kernel(T *__restrict__ delta, T *__restrict__ prev, T *__restrict__ trunc,
                      int32_t *__restrict__ mask, float thr_f, int mode, int P, int C, int lg) {
    constexpr int N = Vec16<T>::N;
    __shared__ int s_list[4][WAVE];
    const int G = 1 << lg;
    const int wave = wave_id(), lane = lane_id();
    const int pm = (blockIdx.x * 4 + wave) * WAVE + lane;
    const bool on = pm < P && mask[min(pm, P - 1)] != 0;
    const uint64_t bits = ballot(on);
    if (bits == 0) return;
    const int n = __popcll((unsigned long long)bits);
    if (on) s_list[wave][__popcll((unsigned long long)(bits & ((1ull << lane) - 1ull)))] = pm;
    const int gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    constexpr int U = 2;  // pixels per group and pass: their loads are in flight together
    for (int k = 0; k < n; k += U * ppi) {  // n is wave-uniform
        Vec<T, N> dl[U][1], q[U][1], tr[U][1];
        bool valid[U];
        size_t p[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp;
            valid[u] = idx < n;
            p[u] = (size_t)s_list[wave][min(idx, n - 1)];
            if (valid[u] && gl * N < C) dl[u][0] = vload<T, N>(delta + p[u] * C + gl * N);
            load_state<T, 1>(q[u], tr[u], valid[u], p[u], gl, G, C, prev, trunc);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (k + u * ppi < n)  // wave-uniform
                act_trunc_pixel<T, 1, ACT>(dl[u], q[u], tr[u], valid[u], p[u], gl, G, C, delta, prev, trunc, mask,
                                           T(thr_f), mode);
    }
}

// Any C / alignment: scalar, two passes (decide, then recompute and write).
template <typename T>
__global__ void __launch_bounds__(256)
act_trunc_gen_kernel(T *__restrict__ delta, T *__restrict__ prev, T *__restrict__ trunc,
                     int32_t *__restrict__ mask, float thr_f, int act, int mode, int P, int C,
                     int lg) {
    const T thr = T(thr_f);
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    const bool valid = p < P && mask[p] != 0;
    if (ballot(valid) == 0) return;
    bool hit = false;
    float sq = 0.f;
    if (valid) {
        for (int c = gl; c < C; c += G) {
            size_t off = (size_t)p * C + c;
            T q = prev[off];
            T t = trunc[off] + delta[off];
            T s = t + q;
            T d = act_apply<T>(s, act) - act_apply<T>(q, act);
            hit |= tabs(d) > thr;
            sq += float(d) * float(d);
        }
    }
    bool keep;
    if (mode == DC_TRUNC_MAX) {
        keep = group_any(hit, G);
    } else {
        sq = group_sum(sq, G);
        if (mode == DC_TRUNC_RMS) sq /= float(C);
        keep = sqrtf(sq) > float(thr);
    }
    if (valid) {
        for (int c = gl; c < C; c += G) {
            size_t off = (size_t)p * C + c;
            T q = prev[off];
            T t = trunc[off] + delta[off];
            if (keep) {
                T s = t + q;
                prev[off] = s;
                delta[off] = act_apply<T>(s, act) - act_apply<T>(q, act);
                trunc[off] = T(0);
            } else {
                trunc[off] = t;
            }
        }
        if (!keep && gl == 0) mask[p] = 0;
    }
}

// -------------------------------------------------------------------------------- densify
// Truncation mode < 0: prev += delta on active pixels; a non-linear activation also rewrites
// delta = act(prev_new) - act(prev_old).
template <typename T, int N>
__global__ void __launch_bounds__(256)
accumulate_kernel(T *__restrict__ delta, T *__restrict__ prev, const int32_t *__restrict__ mask,
                  int act, int P, int C, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P || mask[p] == 0) return;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> dl = vload<T, N>(delta + off);
        Vec<T, N> q = vload<T, N>(prev + off);
        Vec<T, N> s;
#pragma unroll
        for (int j = 0; j < N; ++j) s.v[j] = dl.v[j] + q.v[j];
        vstore<T, N>(prev + off, s);
        if (act > 0) {
#pragma unroll
            for (int j = 0; j < N; ++j)
                dl.v[j] = act_apply<T>(s.v[j], act) - act_apply<T>(q.v[j], act);
            vstore<T, N>(delta + off, dl);
        }
    }
}

// Densify: prev += delta on active pixels, out = prev on every pixel.
template <typename T, int N>
__global__ void __launch_bounds__(256)
densify_kernel(const T *__restrict__ delta, T *__restrict__ prev, T *__restrict__ out,
               const int32_t *__restrict__ mask, int P, int C, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool on = mask[p] != 0;
    for (int c = gl * N; c < C; c += G * N) {
        const size_t off = (size_t)p * C + c;
        Vec<T, N> q = vload<T, N>(prev + off);
        if (on) {
            const Vec<T, N> dl = vload<T, N>(delta + off);
#pragma unroll
            for (int j = 0; j < N; ++j) q.v[j] = dl.v[j] + q.v[j];
            vstore<T, N>(prev + off, q);
        }
        vstore<T, N>(out + off, q);
    }
}

// ------------------------------------------------------------------------------------ add
// s = wa*a*[Ma]; s = fma(b, wb, s)*[Mb]; mask_out = Ma | Mb (written for every pixel).
// act > 0: prev += s, out = act(prev_new) - act(prev_old).
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ prev,
           T *__restrict__ out, const int32_t *__restrict__ ma, const int32_t *__restrict__ mb,
           int32_t *__restrict__ mo, float wa_f, float wb_f, int act, int P, int C, int lg) {
    const T wa = T(wa_f), wb = T(wb_f);
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool aa = ma[p] != 0, ab = mb[p] != 0;
    if (gl == 0) mo[p] = (aa || ab) ? 1 : 0;
    if (!(aa || ab)) return;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> s;
#pragma unroll
        for (int j = 0; j < N; ++j) s.v[j] = T(0);
        if (aa) {
            Vec<T, N> va = vload<T, N>(a + off);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = va.v[j] * wa;
        }
        if (ab) {
            Vec<T, N> vb = vload<T, N>(b + off);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = fma_t(vb.v[j], wb, s.v[j]);
        }
        if (act > 0) {
            Vec<T, N> q = vload<T, N>(prev + off);
            Vec<T, N> n;
#pragma unroll
            for (int j = 0; j < N; ++j) {
                n.v[j] = s.v[j] + q.v[j];
                s.v[j] = act_apply<T>(n.v[j], act) - act_apply<T>(q.v[j], act);
            }
            vstore<T, N>(prev + off, n);
        }
        vstore<T, N>(out + off, s);
    }
}

// add_kernel whose second operand lives on a map S times smaller in both directions and is
// read through nearest upsampling: pixel (y, x) takes b and its mask word at (y / S, x / S).
// The upsampled tensor never exists in memory.
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_up_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ prev,
              T *__restrict__ out, const int32_t *__restrict__ ma, const int32_t *__restrict__ mb,
              int32_t *__restrict__ mo, float wa_f, float wb_f, int act, int B, int H, int W, int C,
              int S, int lg) {
    const T wa = T(wa_f), wb = T(wb_f);
    const int G = 1 << lg, P = B * H * W;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const int row = p / W, x = p - row * W;  // row = image * H + y
    const int img = row / H, y = row - img * H;
    const size_t pb = ((size_t)img * (H / S) + y / S) * (W / S) + x / S;
    const bool aa = ma[p] != 0, ab = mb[pb] != 0;
    if (gl == 0) mo[p] = (aa || ab) ? 1 : 0;
    if (!(aa || ab)) return;
    for (int c = gl * N; c < C; c += G * N) {
        const size_t off = (size_t)p * C + c;
        Vec<T, N> s;
#pragma unroll
        for (int j = 0; j < N; ++j) s.v[j] = T(0);
        if (aa) {
            Vec<T, N> va = vload<T, N>(a + off);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = va.v[j] * wa;
        }
        if (ab) {
            Vec<T, N> vb = vload<T, N>(b + pb * C + c);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = fma_t(vb.v[j], wb, s.v[j]);
        }
        if (act > 0) {
            Vec<T, N> q = vload<T, N>(prev + off);
            Vec<T, N> n;
#pragma unroll
            for (int j = 0; j < N; ++j) {
                n.v[j] = s.v[j] + q.v[j];
                s.v[j] = act_apply<T>(n.v[j], act) - act_apply<T>(q.v[j], act);
            }
            vstore<T, N>(prev + off, n);
        }
        vstore<T, N>(out + off, s);
    }
}

// Several independent sums in one launch (the sums of one level of a multi-resolution exchange):
// a workgroup looks up the sum its number falls into; a plain sum is an upsampled one of scale 1.
// The arithmetic is add_up_kernel's, element by element.
template <typename T>
struct AddItemD {
    const T *a, *b;
    T *prev, *out;
    const int32_t *ma, *mb;
    int32_t *mo;
    float wa, wb;
    int act, B, H, W, C, S, lg, first;
};

template <typename T>
struct AddGroupD {
    int n;
    AddItemD<T> it[CONV_GROUP_MAX];
};

template <typename T>
__global__ void __launch_bounds__(256)
add_group_kernel(AddGroupD<T> g) {
    constexpr int N = Vec16<T>::N;
    int idx = 0;
#pragma unroll
    for (int i = 1; i < CONV_GROUP_MAX; ++i)
        if (i < g.n && (int)blockIdx.x >= g.it[i].first) idx = i;
    const AddItemD<T> &it = g.it[idx];
    const T wa = T(it.wa), wb = T(it.wb);
    const int G = 1 << it.lg, H = it.H, W = it.W, C = it.C, S = it.S, P = it.B * H * W;
    const int gid = (blockIdx.x - it.first) * 256 + threadIdx.x;
    const int p = gid >> it.lg, gl = gid & (G - 1);
    if (p >= P) return;
    const int row = p / W, x = p - row * W;  // row = image * H + y
    const int img = row / H, y = row - img * H;
    const size_t pb = ((size_t)img * (H / S) + y / S) * (W / S) + x / S;
    const bool aa = it.ma[p] != 0, ab = it.mb[pb] != 0;
    if (gl == 0) it.mo[p] = (aa || ab) ? 1 : 0;
    if (!(aa || ab)) return;
    const int act = it.act;
    for (int c = gl * N; c < C; c += G * N) {
        const size_t off = (size_t)p * C + c;
        Vec<T, N> s;
#pragma unroll
        for (int j = 0; j < N; ++j) s.v[j] = T(0);
        if (aa) {
            Vec<T, N> va = vload<T, N>(it.a + off);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = va.v[j] * wa;
        }
        if (ab) {
            Vec<T, N> vb = vload<T, N>(it.b + pb * C + c);
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = fma_t(vb.v[j], wb, s.v[j]);
        }
        if (act > 0) {
            Vec<T, N> q = vload<T, N>(it.prev + off);
            Vec<T, N> n;
#pragma unroll
            for (int j = 0; j < N; ++j) {
                n.v[j] = s.v[j] + q.v[j];
                s.v[j] = act_apply<T>(n.v[j], act) - act_apply<T>(q.v[j], act);
            }
            vstore<T, N>(it.prev + off, n);
        }
        vstore<T, N>(it.out + off, s);
    }
}

// add_kernel for large maps: mask scan and compaction per wavefront (see act_trunc_scan_kernel).
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_scan_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ prev,
                T *__restrict__ out, const int32_t *__restrict__ ma, const int32_t *__restrict__ mb,
                int32_t *__restrict__ mo, float wa_f, float wb_f, int act, int P, int C, int lg) {
    __shared__ int s_list[4][WAVE];
    const T wa = T(wa_f), wb = T(wb_f);
    const int G = 1 << lg;
    const int wave = wave_id(), lane = lane_id();
    const int p0 = (blockIdx.x * 4 + wave) * WAVE;
    const int pm = p0 + lane;
    const bool la = pm < P && ma[min(pm, P - 1)] != 0, lb = pm < P && mb[min(pm, P - 1)] != 0;
    if (pm < P) mo[pm] = (la || lb) ? 1 : 0;
    const uint64_t bits_a = ballot(la), bits_b = ballot(lb), bits = bits_a | bits_b;
    if (bits == 0) return;
    const int n = __popcll((unsigned long long)bits);
    if (la || lb) s_list[wave][__popcll((unsigned long long)(bits & ((1ull << lane) - 1ull)))] = lane;
    const int gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    constexpr int U = 2;  // pixels per group and pass: their loads are in flight together
    for (int k = 0; k < n; k += U * ppi) {
        for (int c = gl * N; c < C; c += G * N) {
            Vec<T, N> va[U], vb[U], q[U];
            bool aa[U], ab[U], valid[U];
            size_t off[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {  // operands of inactive sides read the row of the other side
                const int idx = k + u * ppi + grp;
                valid[u] = idx < n;
                const int l = s_list[wave][min(idx, n - 1)];
                aa[u] = (bits_a >> l) & 1ull;
                ab[u] = (bits_b >> l) & 1ull;
                off[u] = ((size_t)p0 + l) * C + c;
                va[u] = vload<T, N>((aa[u] ? a : b) + off[u]);
                vb[u] = vload<T, N>((ab[u] ? b : a) + off[u]);
                if (act > 0) q[u] = vload<T, N>(prev + off[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (!valid[u]) continue;
                Vec<T, N> s;
#pragma unroll
                for (int j = 0; j < N; ++j) s.v[j] = aa[u] ? va[u].v[j] * wa : T(0);
                if (ab[u]) {
#pragma unroll
                    for (int j = 0; j < N; ++j) s.v[j] = fma_t(vb[u].v[j], wb, s.v[j]);
                }
                if (act > 0) {
                    Vec<T, N> nn;
#pragma unroll
                    for (int j = 0; j < N; ++j) {
                        nn.v[j] = s.v[j] + q[u].v[j];
                        s.v[j] = act_apply<T>(nn.v[j], act) - act_apply<T>(q[u].v[j], act);
                    }
                    vstore<T, N>(prev + off[u], nn);
                }
                vstore<T, N>(out + off[u], s);
            }
        }
    }
}

// dense_out: prev += s on active pixels, out = act(prev) for every pixel.
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_dense_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ prev,
                 T *__restrict__ out, const int32_t *__restrict__ ma,
                 const int32_t *__restrict__ mb, float wa_f, float wb_f, int act, int P, int C,
                 int lg) {
    const T wa = T(wa_f), wb = T(wb_f);
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool aa = ma[p] != 0, ab = mb[p] != 0;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> q = vload<T, N>(prev + off);
        if (aa || ab) {
            Vec<T, N> s;
#pragma unroll
            for (int j = 0; j < N; ++j) s.v[j] = T(0);
            if (aa) {
                Vec<T, N> va = vload<T, N>(a + off);
#pragma unroll
                for (int j = 0; j < N; ++j) s.v[j] = va.v[j] * wa;
            }
            if (ab) {
                Vec<T, N> vb = vload<T, N>(b + off);
#pragma unroll
                for (int j = 0; j < N; ++j) s.v[j] = fma_t(vb.v[j], wb, s.v[j]);
            }
#pragma unroll
            for (int j = 0; j < N; ++j) q.v[j] = s.v[j] + q.v[j];
            vstore<T, N>(prev + off, q);
        }
#pragma unroll
        for (int j = 0; j < N; ++j) q.v[j] = act_apply<T>(q.v[j], act);
        vstore<T, N>(out + off, q);
    }
}

// --------------------------------------------------------------------------- add to dense
// b[px] += a[px] on active pixels.
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_to_dense_kernel(const T *__restrict__ a, T *__restrict__ b, const int32_t *__restrict__ ma,
                    int P, int C, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P || ma[p] == 0) return;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> va = vload<T, N>(a + off);
        Vec<T, N> vb = vload<T, N>(b + off);
#pragma unroll
        for (int j = 0; j < N; ++j) vb.v[j] = vb.v[j] + va.v[j];
        vstore<T, N>(b + off, vb);
    }
}

// With an activation the operator turns `a` into a dense output: b += a on active pixels,
// then a = act(b) on every pixel.
template <typename T, int N>
__global__ void __launch_bounds__(256)
add_to_dense_act_kernel(T *__restrict__ a, T *__restrict__ b, const int32_t *__restrict__ ma,
                        int act, int P, int C, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool active = ma[p] != 0;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> vb = vload<T, N>(b + off);
        if (active) {
            Vec<T, N> va = vload<T, N>(a + off);
#pragma unroll
            for (int j = 0; j < N; ++j) vb.v[j] = vb.v[j] + va.v[j];
            vstore<T, N>(b + off, vb);
        }
#pragma unroll
        for (int j = 0; j < N; ++j) vb.v[j] = act_apply<T>(vb.v[j], act);
        vstore<T, N>(a + off, vb);
    }
}

// ------------------------------------------------------------------------------- upsample
// One group of lanes per OUTPUT pixel (oy, ox), which copies input pixel (oy / S, ox / S) and its
// mask word: S * S times the parallelism of a group per input pixel, coalesced stores, no loop
// over the S x S block; the repeated reads of an input row come from the caches.
template <typename T, int N>
__global__ void __launch_bounds__(256)
upsample_kernel(const T *__restrict__ in, T *__restrict__ out, const int32_t *__restrict__ mi,
                int32_t *__restrict__ mo, int B, int H, int W, int C, int S, int lg) {
    const int Ho = H * S, Wo = W * S;
    const int P = B * Ho * Wo;
    const int G = 1 << lg;
    int po, gl;
    group_coords(lg, po, gl);
    if (po >= P) return;
    const int row = po / Wo, ox = po - row * Wo;  // row = b * Ho + oy
    const int bb = row / Ho, oy = row - bb * Ho;
    const size_t pi = ((size_t)bb * H + oy / S) * W + ox / S;
    const bool active = mi[pi] != 0;
    if (gl == 0) mo[po] = active ? 1 : 0;
    if (!active) return;
    for (int c = gl * N; c < C; c += G * N) vstore<T, N>(out + (size_t)po * C + c, vload<T, N>(in + pi * C + c));
}

// ---------------------------------------------------------------------------- concatenate
template <typename T, int N>
__global__ void __launch_bounds__(256)
concat_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ out,
              const int32_t *__restrict__ ma, const int32_t *__restrict__ mb,
              int32_t *__restrict__ mo, int P, int Ca, int Cb, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool aa = ma[p] != 0, ab = mb[p] != 0;
    if (gl == 0) mo[p] = (aa || ab) ? 1 : 0;
    if (!(aa || ab)) return;
    T *o = out + (size_t)p * (Ca + Cb);
    Vec<T, N> z;
#pragma unroll
    for (int j = 0; j < N; ++j) z.v[j] = T(0);
    for (int c = gl * N; c < Ca; c += G * N)
        vstore<T, N>(o + c, aa ? vload<T, N>(a + (size_t)p * Ca + c) : z);
    for (int c = gl * N; c < Cb; c += G * N)
        vstore<T, N>(o + Ca + c, ab ? vload<T, N>(b + (size_t)p * Cb + c) : z);
}

// -------------------------------------------------------------------------------- mul_add
template <typename T, int N>
__global__ void __launch_bounds__(256)
mul_add_kernel(const T *in, const int32_t *mask, T *out,  // in == out, mask == mo when in place
               int32_t *mo, const T *__restrict__ scale,
               const T *__restrict__ bias, int P, int C, int lg) {
    const int G = 1 << lg;
    int p, gl;
    group_coords(lg, p, gl);
    if (p >= P) return;
    const bool active = mask[p] != 0;
    if (mo != mask && gl == 0) mo[p] = active ? 1 : 0;
    if (!active) return;
    for (int c = gl * N; c < C; c += G * N) {
        size_t off = (size_t)p * C + c;
        Vec<T, N> v = vload<T, N>(in + off);
        Vec<T, N> sc = vload<T, N>(scale + c);
        if (bias != nullptr) {
            Vec<T, N> bi = vload<T, N>(bias + c);
#pragma unroll
            for (int j = 0; j < N; ++j) v.v[j] = fma_t(v.v[j], sc.v[j], bi.v[j]);
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) v.v[j] = v.v[j] * sc.v[j];
        }
        vstore<T, N>(out + off, v);
    }
}

// ------------------------------------------------------------- large maps: scanning forms
// The four operators above for maps of at least SCAN_MIN_PIXELS pixels (see
// act_trunc_scan_kernel): a wavefront reads 64 mask words, writes the 64 output mask words,
// lists its updated pixels in LDS and then serves them U at a time per lane group, so a sparse
// map costs no wavefront launches for pixels that have nothing to do.  One 16-byte vector per
// lane and pixel: G >= C / N.
template <typename T, int N>
__global__ void __launch_bounds__(256)
mul_add_scan_kernel(const T *in, const int32_t *mask, T *out, int32_t *mo, const T *__restrict__ scale,
                    const T *__restrict__ bias, int P, int C, int lg) {
    __shared__ int s_list[4][WAVE];
    const int wave = wave_id(), lane = lane_id();
    const int pm = (blockIdx.x * 4 + wave) * WAVE + lane;
    const bool on = pm < P && mask[min(pm, P - 1)] != 0;
    if (mo != mask && pm < P) mo[pm] = on ? 1 : 0;
    int n;
    const int rank = wave_rank(on, n);
    if (n == 0) return;
    if (on) s_list[wave][rank] = pm;
    const int G = 1 << lg, gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    const bool mine = gl * N < C;
    const int c = min(gl * N, C - N);
    const Vec<T, N> sc = vload<T, N>(scale + c);
    Vec<T, N> bi;
    if (bias != nullptr) bi = vload<T, N>(bias + c);
    constexpr int U = 4;
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> v[U];
        bool valid[U];
        size_t off[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp;
            valid[u] = idx < n && mine;
            off[u] = (size_t)s_list[wave][min(idx, n - 1)] * C + c;
            v[u] = vload<T, N>(in + off[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
            if (bias != nullptr) {
#pragma unroll
                for (int j = 0; j < N; ++j) v[u].v[j] = fma_t(v[u].v[j], sc.v[j], bi.v[j]);
            } else {
#pragma unroll
                for (int j = 0; j < N; ++j) v[u].v[j] = v[u].v[j] * sc.v[j];
            }
            vstore<T, N>(out + off[u], v[u]);
        }
    }
}

template <typename T, int N>
__global__ void __launch_bounds__(256)
add_to_dense_scan_kernel(const T *__restrict__ a, T *__restrict__ b, const int32_t *__restrict__ ma,
                         int P, int C, int lg) {
    __shared__ int s_list[4][WAVE];
    const int wave = wave_id(), lane = lane_id();
    const int pm = (blockIdx.x * 4 + wave) * WAVE + lane;
    const bool on = pm < P && ma[min(pm, P - 1)] != 0;
    int n;
    const int rank = wave_rank(on, n);
    if (n == 0) return;
    if (on) s_list[wave][rank] = pm;
    const int G = 1 << lg, gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    const bool mine = gl * N < C;
    const int c = min(gl * N, C - N);
    constexpr int U = 2;
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> va[U], vb[U];
        bool valid[U];
        size_t off[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp;
            valid[u] = idx < n && mine;
            off[u] = (size_t)s_list[wave][min(idx, n - 1)] * C + c;
            va[u] = vload<T, N>(a + off[u]);
            vb[u] = vload<T, N>(b + off[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
#pragma unroll
            for (int j = 0; j < N; ++j) vb[u].v[j] = vb[u].v[j] + va[u].v[j];
            vstore<T, N>(b + off[u], vb[u]);
        }
    }
}

// Lane gl of a group copies output vector gl of the Ca + Cb channels: from a, or from b behind it
// (zeros where that side was not updated).
template <typename T, int N>
__global__ void __launch_bounds__(256)
concat_scan_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ out,
                   const int32_t *__restrict__ ma, const int32_t *__restrict__ mb,
                   int32_t *__restrict__ mo, int P, int Ca, int Cb, int lg) {
    __shared__ int s_list[4][WAVE];
    const int wave = wave_id(), lane = lane_id();
    const int p0 = (blockIdx.x * 4 + wave) * WAVE;
    const int pm = p0 + lane;
    const bool la = pm < P && ma[min(pm, P - 1)] != 0, lb = pm < P && mb[min(pm, P - 1)] != 0;
    if (pm < P) mo[pm] = (la || lb) ? 1 : 0;
    const uint64_t bits_a = ballot(la), bits_b = ballot(lb);
    int n;
    const int rank = wave_rank(la || lb, n);
    if (n == 0) return;
    if (la || lb) s_list[wave][rank] = lane;
    const int G = 1 << lg, gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    const bool side_a = gl * N < Ca;
    const bool mine = gl * N < Ca + Cb;
    const int cs = side_a ? gl * N : min(gl * N - Ca, Cb - N);  // channel within the lane's side
    constexpr int U = 4;
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> v[U];
        bool valid[U], have[U];
        size_t po[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp;
            valid[u] = idx < n && mine;
            const int l = s_list[wave][min(idx, n - 1)];
            const bool aa = (bits_a >> l) & 1ull, ab = (bits_b >> l) & 1ull;
            po[u] = (size_t)p0 + l;
            have[u] = side_a ? aa : ab;
            // a side that was not updated is not read: the request goes to the other side's row
            const T *mine_p = side_a ? a + po[u] * Ca + cs : b + po[u] * Cb + cs;
            const T *other_p = side_a ? b + po[u] * Cb : a + po[u] * Ca;
            v[u] = vload<T, N>(have[u] ? mine_p : other_p);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
            if (!have[u]) {
#pragma unroll
                for (int j = 0; j < N; ++j) v[u].v[j] = T(0);
            }
            vstore<T, N>(out + po[u] * (Ca + Cb) + (side_a ? cs : Ca + cs), v[u]);
        }
    }
}

// Scans INPUT pixels; an updated pixel is read once and stored S x S times.
template <typename T, int N>
__global__ void __launch_bounds__(256)
upsample_scan_kernel(const T *__restrict__ in, T *__restrict__ out, const int32_t *__restrict__ mi,
                     int32_t *__restrict__ mo, int B, int H, int W, int C, int S, int lg) {
    __shared__ int s_in[4][WAVE], s_out[4][WAVE];
    const int P = B * H * W, Wo = W * S;
    const int wave = wave_id(), lane = lane_id();
    const int pm = (blockIdx.x * 4 + wave) * WAVE + lane;
    const int pc = min(pm, P - 1);
    const bool on = pm < P && mi[pc] != 0;
    const int row = pc / W, x = pc - row * W;         // row = b * H + y
    const int obase = row * S * Wo + x * S;            // top left output pixel of the block
    if (pm < P) {
        for (int dy = 0; dy < S; ++dy)
            for (int dx = 0; dx < S; ++dx) mo[(size_t)obase + dy * Wo + dx] = on ? 1 : 0;
    }
    int n;
    const int rank = wave_rank(on, n);
    if (n == 0) return;
    if (on) {
        s_in[wave][rank] = pm;
        s_out[wave][rank] = obase;
    }
    const int G = 1 << lg, gl = lane & (G - 1), grp = lane >> lg, ppi = WAVE >> lg;
    const bool mine = gl * N < C;
    const int c = min(gl * N, C - N);
    constexpr int U = 4;
    for (int k = 0; k < n; k += U * ppi) {
        Vec<T, N> v[U];
        bool valid[U];
        size_t ob[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = k + u * ppi + grp;
            valid[u] = idx < n && mine;
            const int e = min(idx, n - 1);
            ob[u] = (size_t)s_out[wave][e];
            v[u] = vload<T, N>(in + (size_t)s_in[wave][e] * C + c);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!valid[u]) continue;
            for (int dy = 0; dy < S; ++dy)
                for (int dx = 0; dx < S; ++dx) vstore<T, N>(out + (ob[u] + (size_t)dy * Wo + dx) * C + c, v[u]);
        }
    }
}

// ---------------------------------------------------------------------------- host helpers
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T>
bool can_vec(int C, std::initializer_list<const void *> ptrs) {
    if (C % Vec16<T>::N != 0) return false;
    for (const void *p : ptrs)
        if (p != nullptr && !aligned16(p)) return false;
    return true;
}

// Launch shape for one group of G lanes per pixel.
struct GroupLaunch {
    int lg, block;
    dim3 grid;
    GroupLaunch(int64_t pixels, int G)
        : lg(log2i(G)), block(group_block(pixels * G)), grid((unsigned)ceil_div64(pixels * G, block)) {}
};

// the scanning kernels: 16-byte vectors, at most one per lane of a wavefront, a large map
inline bool scan_eligible(bool vec, int64_t pixels, int nvec) {
    return vec && nvec >= 1 && nvec <= WAVE && pixels >= SCAN_MIN_PIXELS;
}

template <typename T>
hipError_t sparsify_t(const T *in, T *prev, T *delta, int32_t *mask, float thr, int P, int C,
                      bool ge, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (can_vec<T>(C, {in, prev, delta}) && C / N <= WAVE * 4) {
        int nvec = C / N;
        int G = pick_group(nvec, P, 4);
        int iters = ceil_div(nvec, G);
        GroupLaunch L(P, G);
        note_kernel("sparsify_vec_kernel");
        switch (iters) {
            case 1: sparsify_vec_kernel<T, 1><<<L.grid, L.block, 0, s>>>(in, prev, delta, mask, thr, P, C, G, ge); break;
            case 2: sparsify_vec_kernel<T, 2><<<L.grid, L.block, 0, s>>>(in, prev, delta, mask, thr, P, C, G, ge); break;
            default: sparsify_vec_kernel<T, 4><<<L.grid, L.block, 0, s>>>(in, prev, delta, mask, thr, P, C, G, ge); break;
        }
    } else {
        int G = group_lanes(C, 4);
        GroupLaunch L(P, G);
        note_kernel("sparsify_gen_kernel");
        sparsify_gen_kernel<T><<<L.grid, L.block, 0, s>>>(in, prev, delta, mask, thr, P, C, G, ge);
    }
    return hipGetLastError();
}

template <typename T, int ITERS>
void act_trunc_launch(dim3 grid, int block, hipStream_t s, T *delta, T *prev, T *trunc, int32_t *mask,
                      float thr, int act, int mode, int P, int C, int lg) {
    note_kernel("act_trunc_vec_kernel");
    // eager loads where reading the whole map, active or not, costs little
    const bool eager = (int64_t)P * C * (int64_t)sizeof(T) <= (1 << 20);
#define DC_AT(A)                                                                                                    \
    do {                                                                                                            \
        if (eager) act_trunc_vec_kernel<T, ITERS, A, true><<<grid, block, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); \
        else act_trunc_vec_kernel<T, ITERS, A, false><<<grid, block, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg);      \
    } while (0)
    switch (act) {
        case DC_ACT_RELU: DC_AT(DC_ACT_RELU); break;
        case DC_ACT_RELU6: DC_AT(DC_ACT_RELU6); break;
        case DC_ACT_LEAKY: DC_AT(DC_ACT_LEAKY); break;
        case DC_ACT_SIGMOID: DC_AT(DC_ACT_SIGMOID); break;
        case DC_ACT_SWISH: DC_AT(DC_ACT_SWISH); break;
        default: DC_AT(DC_ACT_LINEAR); break;
    }
#undef DC_AT
}

template <typename T>
hipError_t act_trunc_t(T *delta, T *prev, T *trunc, int32_t *mask, float thr, int act, int mode,
                       int P, int C, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (act < 0) act = 0;
    if (mode < 0) {
        if (can_vec<T>(C, {delta, prev})) {
            GroupLaunch L(P, pick_group(C / N, P, 4));
            note_kernel("accumulate_kernel");
            accumulate_kernel<T, N><<<L.grid, L.block, 0, s>>>(delta, prev, mask, act, P, C, L.lg);
        } else {
            GroupLaunch L(P, group_lanes(C, 1));
            note_kernel("accumulate_kernel");
            accumulate_kernel<T, 1><<<L.grid, L.block, 0, s>>>(delta, prev, mask, act, P, C, L.lg);
        }
        return hipGetLastError();
    }
    if (can_vec<T>(C, {delta, prev, trunc}) && C / N <= WAVE * 4) {
        int nvec = C / N;
        const int wide = mode == DC_TRUNC_MAX ? wide_group(nvec, P) : 0;
        int G = wide ? wide : pick_group(nvec, P, 4);
        int iters = ceil_div(nvec, G);
        if (P >= SCAN_MIN_PIXELS && nvec <= WAVE) {
            G = group_lanes(nvec, 1);
            const int lg = log2i(G);
            dim3 grid((unsigned)ceil_div(P, 4 * WAVE));
            note_kernel("act_trunc_scan_kernel");
            switch (act) {
                case DC_ACT_RELU: act_trunc_scan_kernel<T, DC_ACT_RELU><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
                case DC_ACT_RELU6: act_trunc_scan_kernel<T, DC_ACT_RELU6><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
                case DC_ACT_LEAKY: act_trunc_scan_kernel<T, DC_ACT_LEAKY><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
                case DC_ACT_SIGMOID: act_trunc_scan_kernel<T, DC_ACT_SIGMOID><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
                case DC_ACT_SWISH: act_trunc_scan_kernel<T, DC_ACT_SWISH><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
                default: act_trunc_scan_kernel<T, DC_ACT_LINEAR><<<grid, 256, 0, s>>>(delta, prev, trunc, mask, thr, mode, P, C, lg); break;
            }
            return hipGetLastError();
        }
        GroupLaunch L(P, G);
        if (wide) {  // one pixel per workgroup
            L.block = wide;
            L.grid = dim3((unsigned)P);
        }
        switch (iters) {
            case 1: act_trunc_launch<T, 1>(L.grid, L.block, s, delta, prev, trunc, mask, thr, act, mode, P, C, L.lg); break;
            case 2: act_trunc_launch<T, 2>(L.grid, L.block, s, delta, prev, trunc, mask, thr, act, mode, P, C, L.lg); break;
            default: act_trunc_launch<T, 4>(L.grid, L.block, s, delta, prev, trunc, mask, thr, act, mode, P, C, L.lg); break;
        }
    } else {
        GroupLaunch L(P, group_lanes(C, 1));
        note_kernel("act_trunc_gen_kernel");
        act_trunc_gen_kernel<T><<<L.grid, L.block, 0, s>>>(delta, prev, trunc, mask, thr, act, mode, P, C, L.lg);
    }
    return hipGetLastError();
}

template <typename T>
hipError_t add_t(const T *a, const T *b, T *prev, T *out, const int32_t *ma, const int32_t *mb,
                 int32_t *mo, float wa, float wb, int act, bool dense_out, int P, int C,
                 hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (act < 0) act = 0;
    const bool vec = can_vec<T>(C, {a, b, prev, out});
    if (!dense_out && vec && P >= SCAN_MIN_PIXELS) {
        const int lg = log2i(group_lanes(C / N, 1));
        note_kernel("add_scan_kernel");
        add_scan_kernel<T, N><<<dim3((unsigned)ceil_div(P, 4 * WAVE)), 256, 0, s>>>(a, b, prev, out, ma, mb, mo, wa, wb, act, P, C, lg);
        return hipGetLastError();
    }
    GroupLaunch L(P, vec ? pick_group(C / N, P, 4) : group_lanes(C, 1));
    note_kernel(dense_out ? "add_dense_kernel" : "add_kernel");
    if (dense_out) {
        if (vec) add_dense_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, wa, wb, act, P, C, L.lg);
        else add_dense_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, wa, wb, act, P, C, L.lg);
    } else {
        if (vec) add_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, mo, wa, wb, act, P, C, L.lg);
        else add_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, mo, wa, wb, act, P, C, L.lg);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_sparsify(const void *in, void *prev, void *delta, int32_t *mask, float thr,
                           int32_t P, int32_t C, int dtype, hipStream_t s) {
    if (dtype == DC_F32)
        return sparsify_t<float>((const float *)in, (float *)prev, (float *)delta, mask, thr, P, C, false, s);
    if (dtype == DC_BF16)
        return sparsify_t<bf16_t>((const bf16_t *)in, (bf16_t *)prev, (bf16_t *)delta, mask, thr, P, C, false, s);
    return sparsify_t<half_t>((const half_t *)in, (half_t *)prev, (half_t *)delta, mask, thr, P, C,
                              C % 2 == 0, s);
}

hipError_t launch_activate_truncate(void *delta, void *prev, void *trunc, int32_t *mask, float thr,
                                    int act, int mode, int32_t P, int32_t C, int dtype,
                                    hipStream_t s) {
    if (dtype == DC_F32)
        return act_trunc_t<float>((float *)delta, (float *)prev, (float *)trunc, mask, thr, act, mode, P, C, s);
    if (dtype == DC_BF16)
        return act_trunc_t<bf16_t>((bf16_t *)delta, (bf16_t *)prev, (bf16_t *)trunc, mask, thr, act, mode, P, C, s);
    return act_trunc_t<half_t>((half_t *)delta, (half_t *)prev, (half_t *)trunc, mask, thr, act, mode, P, C, s);
}

// 16-byte rows, at most four vectors per lane of a 64-lane group, tensors of at most 1 MB (the
// eager form reads every pixel's row).
bool act_group_eligible(const ActGroupItem *items, int n, int act, int mode, int dtype) {
    if (n < 1 || n > CONV_GROUP_MAX || mode != DC_TRUNC_MAX || act > DC_ACT_SWISH) return false;
    if (dtype != DC_F16 && dtype != DC_BF16) return false;
    for (int i = 0; i < n; ++i) {
        const ActGroupItem &a = items[i];
        if (a.P <= 0 || a.C <= 0 || a.C % 8 != 0 || a.C / 8 > WAVE * 4) return false;
        if ((int64_t)a.P * a.C * 2 > (1 << 20)) return false;
        for (const void *q : {(const void *)a.delta, (const void *)a.prev, (const void *)a.trunc})
            if (q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15u) != 0) return false;
        if (a.mask == nullptr) return false;
    }
    return true;
}

namespace {
template <typename T>
hipError_t act_group_t(const ActGroupItem *items, int n, int act, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    ActGroupD<T> ag;
    ag.n = n;
    int blocks = 0;
    for (int i = 0; i < n; ++i) {
        const ActGroupItem &a = items[i];
        ActItemD<T> &it = ag.it[i];
        const int nvec = a.C / N;
        const int G = pick_group(nvec, a.P, 4);
        it.delta = (T *)a.delta; it.prev = (T *)a.prev; it.trunc = (T *)a.trunc; it.mask = a.mask;
        it.thr = a.thr; it.P = a.P; it.C = a.C;
        it.lg = log2i(G);
        const int iters = ceil_div(nvec, G);
        it.iters = iters <= 1 ? 1 : iters <= 2 ? 2 : 4;
        it.first = blocks;
        blocks += (int)ceil_div64((int64_t)a.P * G, 256);
    }
    for (int i = n; i < CONV_GROUP_MAX; ++i) ag.it[i] = ag.it[0];
    note_kernel("act_trunc_group_kernel");
    const dim3 grid((unsigned)blocks);
    if (act < 0) act = 0;
    switch (act) {
        case DC_ACT_RELU: act_trunc_group_kernel<T, DC_ACT_RELU><<<grid, 256, 0, s>>>(ag); break;
        case DC_ACT_RELU6: act_trunc_group_kernel<T, DC_ACT_RELU6><<<grid, 256, 0, s>>>(ag); break;
        case DC_ACT_LEAKY: act_trunc_group_kernel<T, DC_ACT_LEAKY><<<grid, 256, 0, s>>>(ag); break;
        case DC_ACT_SIGMOID: act_trunc_group_kernel<T, DC_ACT_SIGMOID><<<grid, 256, 0, s>>>(ag); break;
        case DC_ACT_SWISH: act_trunc_group_kernel<T, DC_ACT_SWISH><<<grid, 256, 0, s>>>(ag); break;
        default: act_trunc_group_kernel<T, DC_ACT_LINEAR><<<grid, 256, 0, s>>>(ag); break;
    }
    return hipGetLastError();
}
}  // namespace

hipError_t launch_activate_truncate_group(const ActGroupItem *items, int n, int act, int dtype, hipStream_t s) {
    if (dtype == DC_BF16) return act_group_t<bf16_t>(items, n, act, s);
    return act_group_t<half_t>(items, n, act, s);
}

template <typename T>
hipError_t densify_t(const T *delta, T *prev, T *out, const int32_t *mask, int P, int C, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (can_vec<T>(C, {delta, prev, out})) {
        GroupLaunch L(P, pick_group(C / N, P, 4));
        note_kernel("densify_kernel");
        densify_kernel<T, N><<<L.grid, L.block, 0, s>>>(delta, prev, out, mask, P, C, L.lg);
    } else {
        GroupLaunch L(P, group_lanes(C, 1));
        note_kernel("densify_kernel");
        densify_kernel<T, 1><<<L.grid, L.block, 0, s>>>(delta, prev, out, mask, P, C, L.lg);
    }
    return hipGetLastError();
}

hipError_t launch_densify(const void *delta, void *prev, void *out, const int32_t *mask, int P, int C,
                          int dtype, hipStream_t s) {
    if (dtype == DC_F32) return densify_t<float>((const float *)delta, (float *)prev, (float *)out, mask, P, C, s);
    if (dtype == DC_BF16)
        return densify_t<bf16_t>((const bf16_t *)delta, (bf16_t *)prev, (bf16_t *)out, mask, P, C, s);
    return densify_t<half_t>((const half_t *)delta, (half_t *)prev, (half_t *)out, mask, P, C, s);
}

namespace {
template <typename T>
hipError_t add_up_t(const T *a, const T *b, T *prev, T *out, const int32_t *ma, const int32_t *mb,
                    int32_t *mo, float wa, float wb, int act, int B, int H, int W, int C, int S,
                    hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (act < 0) act = 0;
    const int P = B * H * W;
    const bool vec = can_vec<T>(C, {a, b, prev, out});
    GroupLaunch L(P, vec ? pick_group(C / N, P, 4) : group_lanes(C, 1));
    note_kernel("add_up_kernel");
    if (vec) add_up_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, mo, wa, wb, act, B, H, W, C, S, L.lg);
    else add_up_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, prev, out, ma, mb, mo, wa, wb, act, B, H, W, C, S, L.lg);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_add_upsampled(const void *a, const void *b, void *prev, void *out, const int32_t *ma,
                                const int32_t *mb, int32_t *mo, float wa, float wb, int act, int32_t B,
                                int32_t H, int32_t W, int32_t C, int32_t scale, int dtype, hipStream_t s) {
    if (dtype == DC_F32)
        return add_up_t<float>((const float *)a, (const float *)b, (float *)prev, (float *)out, ma, mb, mo, wa, wb, act, B, H, W, C, scale, s);
    if (dtype == DC_BF16)
        return add_up_t<bf16_t>((const bf16_t *)a, (const bf16_t *)b, (bf16_t *)prev, (bf16_t *)out, ma, mb, mo, wa, wb, act, B, H, W, C, scale, s);
    return add_up_t<half_t>((const half_t *)a, (const half_t *)b, (half_t *)prev, (half_t *)out, ma, mb, mo, wa, wb, act, B, H, W, C, scale, s);
}

// Sums the grouped kernel takes: 16-bit, 16-byte rows and operands, maps below the scanning kernels' size.
bool add_group_eligible(const AddGroupItem *items, int n, int dtype) {
    if (n < 2 || n > CONV_GROUP_MAX || (dtype != DC_F16 && dtype != DC_BF16)) return false;
    for (int i = 0; i < n; ++i) {
        const AddGroupItem &a = items[i];
        if (a.C % 8 != 0 || (int64_t)a.B * a.H * a.W >= SCAN_MIN_PIXELS) return false;
        for (const void *q : {a.a, a.b, (const void *)a.prev, (const void *)a.out})
            if ((reinterpret_cast<uintptr_t>(q) & 15u) != 0) return false;
    }
    return true;
}

namespace {
template <typename T>
hipError_t add_group_t(const AddGroupItem *items, int n, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    AddGroupD<T> ag;
    ag.n = n;
    int blocks = 0;
    for (int i = 0; i < n; ++i) {
        const AddGroupItem &a = items[i];
        AddItemD<T> &it = ag.it[i];
        const int P = a.B * a.H * a.W;
        it.a = (const T *)a.a; it.b = (const T *)a.b; it.prev = (T *)a.prev; it.out = (T *)a.out;
        it.ma = a.ma; it.mb = a.mb; it.mo = a.mo;
        it.wa = a.wa; it.wb = a.wb; it.act = a.act < 0 ? 0 : a.act;
        it.B = a.B; it.H = a.H; it.W = a.W; it.C = a.C; it.S = a.S;
        it.lg = log2i(pick_group(a.C / N, P, 4));
        it.first = blocks;
        blocks += (int)ceil_div64((int64_t)P << it.lg, 256);
    }
    for (int i = n; i < CONV_GROUP_MAX; ++i) ag.it[i] = ag.it[0];
    note_kernel("add_group_kernel");
    add_group_kernel<T><<<dim3((unsigned)blocks), 256, 0, s>>>(ag);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_add_group(const AddGroupItem *items, int n, int dtype, hipStream_t s) {
    if (dtype == DC_BF16) return add_group_t<bf16_t>(items, n, s);
    return add_group_t<half_t>(items, n, s);
}

hipError_t launch_add(const void *a, const void *b, void *prev, void *out, const int32_t *ma,
                      const int32_t *mb, int32_t *mo, float wa, float wb, int act, int dense_out,
                      int32_t P, int32_t C, int dtype, hipStream_t s) {
    if (dtype == DC_F32)
        return add_t<float>((const float *)a, (const float *)b, (float *)prev, (float *)out, ma, mb, mo, wa, wb, act, dense_out != 0, P, C, s);
    if (dtype == DC_BF16)
        return add_t<bf16_t>((const bf16_t *)a, (const bf16_t *)b, (bf16_t *)prev, (bf16_t *)out, ma, mb, mo, wa, wb, act, dense_out != 0, P, C, s);
    return add_t<half_t>((const half_t *)a, (const half_t *)b, (half_t *)prev, (half_t *)out, ma, mb, mo, wa, wb, act, dense_out != 0, P, C, s);
}

namespace {
template <typename T>
hipError_t add_to_dense_t(T *a, T *b, const int32_t *ma, int act, int P, int C, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    const bool vec = can_vec<T>(C, {a, b});
    if (act <= 0 && scan_eligible(vec, P, C / N)) {
        note_kernel("add_to_dense_scan_kernel");
        add_to_dense_scan_kernel<T, N><<<dim3((unsigned)ceil_div(P, 4 * WAVE)), 256, 0, s>>>(a, b, ma, P, C, log2i(group_lanes(C / N, 1)));
        return hipGetLastError();
    }
    GroupLaunch L(P, vec ? pick_group(C / N, P, 4) : group_lanes(C, 1));
    note_kernel(act > 0 ? "add_to_dense_act_kernel" : "add_to_dense_kernel");
    if (act > 0) {
        if (vec) add_to_dense_act_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, ma, act, P, C, L.lg);
        else add_to_dense_act_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, ma, act, P, C, L.lg);
    } else {
        if (vec) add_to_dense_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, ma, P, C, L.lg);
        else add_to_dense_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, ma, P, C, L.lg);
    }
    return hipGetLastError();
}
template <typename T>
hipError_t upsample_t(const T *in, T *out, const int32_t *mi, int32_t *mo, int B, int H, int W,
                      int C, int S, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    int P = B * H * W * S * S;  // output pixels
    if (scan_eligible(can_vec<T>(C, {in, out}), B * H * W, C / N)) {
        note_kernel("upsample_scan_kernel");
        upsample_scan_kernel<T, N><<<dim3((unsigned)ceil_div(B * H * W, 4 * WAVE)), 256, 0, s>>>(in, out, mi, mo, B, H, W, C, S, log2i(group_lanes(C / N, 1)));
        return hipGetLastError();
    }
    if (can_vec<T>(C, {in, out})) {
        GroupLaunch L(P, pick_group(C / N, P, 4));
        note_kernel("upsample_kernel");
        upsample_kernel<T, N><<<L.grid, L.block, 0, s>>>(in, out, mi, mo, B, H, W, C, S, L.lg);
    } else {
        GroupLaunch L(P, group_lanes(C, 1));
        note_kernel("upsample_kernel");
        upsample_kernel<T, 1><<<L.grid, L.block, 0, s>>>(in, out, mi, mo, B, H, W, C, S, L.lg);
    }
    return hipGetLastError();
}
template <typename T>
hipError_t concat_t(const T *a, const T *b, T *out, const int32_t *ma, const int32_t *mb,
                    int32_t *mo, int P, int Ca, int Cb, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    int Cm = Ca > Cb ? Ca : Cb;
    if (Ca % N == 0 && Cb % N == 0 && scan_eligible(can_vec<T>(Ca, {a, b, out}), P, (Ca + Cb) / N)) {
        note_kernel("concat_scan_kernel");
        concat_scan_kernel<T, N><<<dim3((unsigned)ceil_div(P, 4 * WAVE)), 256, 0, s>>>(a, b, out, ma, mb, mo, P, Ca, Cb, log2i(group_lanes((Ca + Cb) / N, 1)));
        return hipGetLastError();
    }
    if (Ca % N == 0 && Cb % N == 0 && can_vec<T>(Ca, {a, b, out})) {
        GroupLaunch L(P, pick_group(Cm / N, P, 4));
        note_kernel("concat_kernel");
        concat_kernel<T, N><<<L.grid, L.block, 0, s>>>(a, b, out, ma, mb, mo, P, Ca, Cb, L.lg);
    } else {
        GroupLaunch L(P, group_lanes(Cm, 1));
        note_kernel("concat_kernel");
        concat_kernel<T, 1><<<L.grid, L.block, 0, s>>>(a, b, out, ma, mb, mo, P, Ca, Cb, L.lg);
    }
    return hipGetLastError();
}
template <typename T>
hipError_t mul_add_t(const T *in, const int32_t *mask, T *out, int32_t *mo, const T *scale,
                     const T *bias, int P, int C, hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    if (scan_eligible(can_vec<T>(C, {in, out, scale, bias}), P, C / N)) {
        note_kernel("mul_add_scan_kernel");
        mul_add_scan_kernel<T, N><<<dim3((unsigned)ceil_div(P, 4 * WAVE)), 256, 0, s>>>(in, mask, out, mo, scale, bias, P, C, log2i(group_lanes(C / N, 1)));
        return hipGetLastError();
    }
    if (can_vec<T>(C, {in, out, scale, bias})) {
        GroupLaunch L(P, pick_group(C / N, P, 4));
        note_kernel("mul_add_kernel");
        mul_add_kernel<T, N><<<L.grid, L.block, 0, s>>>(in, mask, out, mo, scale, bias, P, C, L.lg);
    } else {
        GroupLaunch L(P, group_lanes(C, 1));
        note_kernel("mul_add_kernel");
        mul_add_kernel<T, 1><<<L.grid, L.block, 0, s>>>(in, mask, out, mo, scale, bias, P, C, L.lg);
    }
    return hipGetLastError();
}
}  // namespace

hipError_t launch_add_to_dense(void *a, void *b, const int32_t *ma, int act, int32_t P, int32_t C,
                               int dtype, hipStream_t s) {
    if (dtype == DC_F32) return add_to_dense_t<float>((float *)a, (float *)b, ma, act, P, C, s);
    if (dtype == DC_BF16)
        return add_to_dense_t<bf16_t>((bf16_t *)a, (bf16_t *)b, ma, act, P, C, s);
    return add_to_dense_t<half_t>((half_t *)a, (half_t *)b, ma, act, P, C, s);
}

hipError_t launch_upsample(const void *in, void *out, const int32_t *mi, int32_t *mo, int32_t B,
                           int32_t H, int32_t W, int32_t C, int32_t scale, int dtype,
                           hipStream_t s) {
    if (dtype == DC_F32) return upsample_t<float>((const float *)in, (float *)out, mi, mo, B, H, W, C, scale, s);
    if (dtype == DC_BF16)
        return upsample_t<bf16_t>((const bf16_t *)in, (bf16_t *)out, mi, mo, B, H, W, C, scale, s);
    return upsample_t<half_t>((const half_t *)in, (half_t *)out, mi, mo, B, H, W, C, scale, s);
}

hipError_t launch_concat(const void *a, const void *b, void *out, const int32_t *ma,
                         const int32_t *mb, int32_t *mo, int32_t P, int32_t Ca, int32_t Cb,
                         int dtype, hipStream_t s) {
    if (dtype == DC_F32) return concat_t<float>((const float *)a, (const float *)b, (float *)out, ma, mb, mo, P, Ca, Cb, s);
    if (dtype == DC_BF16)
        return concat_t<bf16_t>((const bf16_t *)a, (const bf16_t *)b, (bf16_t *)out, ma, mb, mo, P, Ca, Cb, s);
    return concat_t<half_t>((const half_t *)a, (const half_t *)b, (half_t *)out, ma, mb, mo, P, Ca, Cb, s);
}

hipError_t launch_mul_add(const void *in, const int32_t *mask, void *out, int32_t *mo,
                          const void *scale, const void *bias, int32_t P, int32_t C, int dtype,
                          hipStream_t s) {
    if (dtype == DC_F32) return mul_add_t<float>((const float *)in, mask, (float *)out, mo, (const float *)scale, (const float *)bias, P, C, s);
    if (dtype == DC_BF16)
        return mul_add_t<bf16_t>((const bf16_t *)in, mask, (bf16_t *)out, mo, (const bf16_t *)scale, (const bf16_t *)bias, P, C, s);
    return mul_add_t<half_t>((const half_t *)in, mask, (half_t *)out, mo, (const half_t *)scale, (const half_t *)bias, P, C, s);
}

}  // namespace dc
