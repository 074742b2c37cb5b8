// Dense head of a classification network: out[r][o] = bias[o] + sum_i x[r][i] * W[o][i] for a
// handful of rows r (one per video stream), W in the [out_features][in_features] layout of
// torch.nn.Linear.  The reference leaves this to torch (example/mobilenet_deltacnn.py:196-199,
// 225); at one row it is a 2.5 MB matrix-vector product that a GEMM library spends several
// launch latencies on, while the frame around it is a chain of two-microsecond kernels.
//
// One wavefront per output feature: the lanes split the feature's weight row into 16-byte
// vectors (V per lane, all requested before anything is waited for, together with the matching
// vectors of up to ROWS input rows), accumulate in fp32 and combine over the wavefront with a
// fixed butterfly, so the sum has one order and needs no atomics.  One rounding to the output
// type after the bias.
#include "common.hpp"

namespace dc {
namespace {

constexpr int LIN_ROWS = 8;  // input rows per workgroup (grid.y covers the rest)

template <typename T, int V>
__global__ void __launch_bounds__(256)
linear_kernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
              T *__restrict__ out, int rows, int in_f, int out_f) {
    constexpr int N = Vec16<T>::N;
    const int o = blockIdx.x * 4 + wave_id();
    if (o >= out_f) return;
    const int lane = lane_id();
    const int r0 = blockIdx.y * LIN_ROWS;
    const int nr = min(LIN_ROWS, rows - r0);
    const int nvec = in_f / N;
    const T *wr = w + (size_t)o * in_f;
    float acc[LIN_ROWS];
#pragma unroll
    for (int r = 0; r < LIN_ROWS; ++r) acc[r] = 0.f;
    for (int base = 0; base < nvec; base += WAVE * V) {
        Vec<T, N> wv[V];
        int vi[V];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            vi[k] = base + k * WAVE + lane;
            wv[k] = vload<T, N>(wr + (size_t)min(vi[k], nvec - 1) * N);
        }
#pragma unroll
        for (int r = 0; r < LIN_ROWS; ++r) {
            if (r >= nr) break;  // uniform
            Vec<T, N> xv[V];
#pragma unroll
            for (int k = 0; k < V; ++k)
                xv[k] = vload<T, N>(x + (size_t)(r0 + r) * in_f + (size_t)min(vi[k], nvec - 1) * N);
#pragma unroll
            for (int k = 0; k < V; ++k) {
                if (vi[k] < nvec) {
#pragma unroll
                    for (int j = 0; j < N; ++j) acc[r] = fmaf(float(xv[k].v[j]), float(wv[k].v[j]), acc[r]);
                }
            }
        }
    }
    const float bv = bias != nullptr ? float(bias[o]) : 0.f;
#pragma unroll
    for (int r = 0; r < LIN_ROWS; ++r) {
        if (r >= nr) break;
        float s = acc[r];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, WAVE);
        if (lane == 0) out[(size_t)(r0 + r) * out_f + o] = T(s + bv);
    }
}

template <typename T>
hipError_t linear_t(const T *x, const T *w, const T *bias, T *out, int rows, int in_f, int out_f,
                    hipStream_t s) {
    constexpr int N = Vec16<T>::N;
    const int per_lane = ceil_div(in_f / N, WAVE);
    dim3 grid(ceil_div(out_f, 4), ceil_div(rows, LIN_ROWS));
    note_kernel("linear_kernel");
    if (per_lane <= 1) linear_kernel<T, 1><<<grid, 256, 0, s>>>(x, w, bias, out, rows, in_f, out_f);
    else if (per_lane == 2) linear_kernel<T, 2><<<grid, 256, 0, s>>>(x, w, bias, out, rows, in_f, out_f);
    else if (per_lane == 3) linear_kernel<T, 3><<<grid, 256, 0, s>>>(x, w, bias, out, rows, in_f, out_f);
    else linear_kernel<T, 4><<<grid, 256, 0, s>>>(x, w, bias, out, rows, in_f, out_f);
    return hipGetLastError();
}

}  // namespace

bool linear_eligible(int in_f, int dtype) {
    const int n = dtype == DC_F32 ? 4 : 8;
    return in_f >= n && in_f % n == 0;
}

hipError_t launch_linear(const void *x, const void *w, const void *bias, void *out, int rows, int in_f,
                         int out_f, int dtype, hipStream_t s) {
    if (dtype == DC_F32)
        return linear_t<float>((const float *)x, (const float *)w, (const float *)bias, (float *)out, rows, in_f, out_f, s);
    if (dtype == DC_BF16)
        return linear_t<bf16_t>((const bf16_t *)x, (const bf16_t *)w, (const bf16_t *)bias, (bf16_t *)out, rows, in_f, out_f, s);
    return linear_t<half_t>((const half_t *)x, (const half_t *)w, (const half_t *)bias, (half_t *)out, rows, in_f, out_f, s);
}

}  // namespace dc
