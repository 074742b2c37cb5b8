// Shared device helpers and the internal launch interface of libdeltacnn_hip.so.
// gfx950 only: wavefronts are 64 lanes wide and every kernel here relies on that.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/deltacnn_hip.h"

namespace dc {

constexpr int WAVE = 64;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16_t;
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// The two 16-bit element types of the matrix-core kernels: vector types and the MFMA
// instruction (16 x 16 outputs, 32 reduction elements, fp32 accumulate).
template <typename E>
struct Elem16;
template <>
struct Elem16<half_t> {
    typedef half4_t v4;
    typedef half8_t v8;
    static __device__ __forceinline__ float4_t mfma(v8 a, v8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Elem16<bf16_t> {
    typedef bf16x4_t v4;
    typedef bf16x8_t v8;
    static __device__ __forceinline__ float4_t mfma(v8 a, v8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <typename E>
__device__ __forceinline__ typename Elem16<E>::v4 zero4() {
    return typename Elem16<E>::v4{E(0), E(0), E(0), E(0)};
}

// N elements of T moved with one naturally aligned load / store.
template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
    T v[N];
};

template <typename T, int N>
__device__ __forceinline__ Vec<T, N> vload(const T *p) {
    return *reinterpret_cast<const Vec<T, N> *>(p);
}
template <typename T, int N>
__device__ __forceinline__ void vstore(T *p, const Vec<T, N> &x) {
    *reinterpret_cast<Vec<T, N> *>(p) = x;
}

// DC_PIN (below) for a 16-byte Vec: the load that produced `x` is issued before this program
// point instead of where the compiler would sink it to -- next to its first use, possibly behind
// a barrier or a run of stores, where its latency would be paid on its own.  Place it where
// the value has arrived anyway (behind a wait for a request issued later).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <typename T, int N>
__device__ __forceinline__ void pin_vec(Vec<T, N> &x) {
    static_assert(sizeof(Vec<T, N>) == 16, "16-byte vectors only");
    union {
        Vec<T, N> v;
        u32x4_t r;
    } c;
    c.v = x;
    asm volatile("" : "+v"(c.r));
    x = c.v;
}

// Largest magnitude of a 16-byte vector's elements (NaN elements are skipped, as a comparison
// against a threshold would skip them); halves take the packed instructions.
__device__ __forceinline__ float vec_absmax(const Vec<half_t, 8> &x) {
    union {
        Vec<half_t, 8> v;
        half8_t h;
    } c;
    c.v = x;
    const half8_t a = __builtin_elementwise_abs(c.h);
    const half4_t m4 = __builtin_elementwise_max(a.lo, a.hi);
    const half2_t m2 = __builtin_elementwise_max(m4.lo, m4.hi);
    return float(__builtin_fmaxf16(m2[0], m2[1]));
}
template <typename T, int N>
__device__ __forceinline__ float vec_absmax(const Vec<T, N> &x) {
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < N; ++j) m = fmaxf(m, __builtin_fabsf(float(x.v[j])));
    return m;
}

// Is any bit of a 16-byte / 8-byte vector set?  (A truncated remainder that is zero already need
// not be stored as zero again.)
template <typename V>
__device__ __forceinline__ bool bits_set16(const V &x) {
    static_assert(sizeof(V) == 16, "16-byte vectors");
    const u32x4_t u = __builtin_bit_cast(u32x4_t, x);
    return ((u[0] | u[1]) | (u[2] | u[3])) != 0u;
}
template <typename V>
__device__ __forceinline__ bool bits_set8(const V &x) {
    static_assert(sizeof(V) == 8, "8-byte vectors");
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    const u32x2_t u = __builtin_bit_cast(u32x2_t, x);
    return (u[0] | u[1]) != 0u;
}

// Is any bit of a 16-byte vector set?
template <typename T, int N>
__device__ __forceinline__ bool any_bits(const Vec<T, N> &x) {
    static_assert(sizeof(Vec<T, N>) == 16, "16-byte vectors only");
    union {
        Vec<T, N> v;
        uint32_t u[4];
    } c;
    c.v = x;
    return ((c.u[0] | c.u[1]) | (c.u[2] | c.u[3])) != 0u;
}

// A 16-byte vector kept if `on`, else all-zero bits: four 32-bit selects whatever the element
// type (a per-element select on halves costs twice as many instructions).
template <typename T, int N>
__device__ __forceinline__ Vec<T, N> vkeep(const Vec<T, N> &x, bool on) {
    static_assert(sizeof(Vec<T, N>) == 16, "16-byte vectors only");
    union {
        Vec<T, N> v;
        uint32_t u[4];
    } c;
    c.v = x;
#pragma unroll
    for (int k = 0; k < 4; ++k) c.u[k] = on ? c.u[k] : 0u;
    return c.v;
}

// The same for an MFMA operand fragment of 8 halves.
__device__ __forceinline__ half8_t keep8(half8_t x, bool on) {
    union {
        half8_t v;
        uint32_t u[4];
    } c;
    c.v = x;
#pragma unroll
    for (int k = 0; k < 4; ++k) c.u[k] = on ? c.u[k] : 0u;
    return c.v;
}

__device__ __forceinline__ bf16x8_t keep8(bf16x8_t x, bool on) {
    union {
        bf16x8_t v;
        uint32_t u[4];
    } c;
    c.v = x;
#pragma unroll
    for (int k = 0; k < 4; ++k) c.u[k] = on ? c.u[k] : 0u;
    return c.v;
}

// Elements per 16-byte vector.
template <typename T>
struct Vec16 {
    static constexpr int N = 16 / sizeof(T);
};

// Pin a loaded value at this program point: the compiler may neither sink the load that
// produced it below this point nor start consuming it earlier, so a run of loads followed by
// a run of pins is issued back to back and waited for once.
#define DC_PIN(x) asm volatile("" : "+v"(x))

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

// Index of the wavefront inside its workgroup, as a scalar: the compiler cannot see that
// threadIdx.x / 64 is the same in all lanes, and would keep everything derived from it
// (step counters, filter addresses, loop conditions) in vector registers and masked branches.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE); }

__device__ __forceinline__ uint64_t ballot(bool p) { return __ballot(p); }

// Does any lane of this lane's aligned group of `g` lanes (g a power of two) hold `p`?
__device__ __forceinline__ bool group_any(bool p, int g) {
    uint64_t b = ballot(p);
    if (g >= WAVE) return b != 0;
    int lo = lane_id() & ~(g - 1);
    return ((b >> lo) & ((1ull << g) - 1ull)) != 0;
}

// Rank of this lane among the lanes with `p` set, and their count.
__device__ __forceinline__ int wave_rank(bool p, int &count) {
    uint64_t b = ballot(p);
    count = __popcll(b);
    return __popcll(b & ((1ull << lane_id()) - 1ull));
}

// Activation functions, one IEEE operation at a time in the tensor's own type so that
// results are bit-identical to evaluating the same expression op by op on the host.
// sigmoid / swish through fp32 exp.  Kept out of line, conversion included: when these are
// inlined into unrolled vector loops the compiler folds the surrounding negations into packed
// two-float operations that this target (packed fp32 ops disabled) cannot select.
__device__ __attribute__((noinline)) float sigmoid_t(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __attribute__((noinline)) float swish_t(float x) { return x * (1.0f / (1.0f + expf(-x))); }
__device__ __attribute__((noinline)) half_t sigmoid_t(half_t x) {
    return half_t(1.0f / (1.0f + expf(-float(x))));
}
__device__ __attribute__((noinline)) half_t swish_t(half_t x) {
    return half_t(float(x) * (1.0f / (1.0f + expf(-float(x)))));
}
__device__ __attribute__((noinline)) bf16_t sigmoid_t(bf16_t x) {
    return bf16_t(1.0f / (1.0f + expf(-float(x))));
}
__device__ __attribute__((noinline)) bf16_t swish_t(bf16_t x) {
    return bf16_t(float(x) * (1.0f / (1.0f + expf(-float(x)))));
}

// max / min as single instructions (v_max_f16, v_max_f32, ...).  For finite operands they give
// the values of the compare-and-select form `x < 0 ? 0 : x`; the two differ only for NaN (here
// replaced by the other operand) and in the sign of a zero result, and NaN never reaches an
// active pixel.
__device__ __forceinline__ float tmax(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ float tmin(float a, float b) { return __builtin_fminf(a, b); }
__device__ __forceinline__ half_t tmax(half_t a, half_t b) { return __builtin_fmaxf16(a, b); }
__device__ __forceinline__ half_t tmin(half_t a, half_t b) { return __builtin_fminf16(a, b); }
// bfloat16 arithmetic is fp32 arithmetic on the widened operands followed by one rounding
// (v_cvt_pk_bf16_f32); max / min / abs of bfloat16 values are exact in either type
__device__ __forceinline__ bf16_t tmax(bf16_t a, bf16_t b) { return bf16_t(__builtin_fmaxf(float(a), float(b))); }
__device__ __forceinline__ bf16_t tmin(bf16_t a, bf16_t b) { return bf16_t(__builtin_fminf(float(a), float(b))); }

template <typename T>
__device__ __forceinline__ T act_apply(T x, int act) {
    switch (act) {
        case DC_ACT_RELU: return tmax(x, T(0));
        case DC_ACT_RELU6: return tmin(tmax(x, T(0)), T(6));
        case DC_ACT_LEAKY: return x < T(0) ? x * T(0.1f) : x;
        case DC_ACT_SIGMOID: return sigmoid_t(x);
        case DC_ACT_SWISH: return swish_t(x);
        default: return x;
    }
}

// Fused multiply-add with a single rounding in the operand type.
__device__ __forceinline__ float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ half_t fma_t(half_t a, half_t b, half_t c) {
    return __builtin_fmaf16(a, b, c);
}
// the fp32 fused multiply-add of bfloat16 operands is exact up to its own rounding (the product
// has 16 significant bits), then rounded to bfloat16
__device__ __forceinline__ bf16_t fma_t(bf16_t a, bf16_t b, bf16_t c) {
    return bf16_t(__builtin_fmaf(float(a), float(b), float(c)));
}

__device__ __forceinline__ float tabs(float x) { return __builtin_fabsf(x); }
__device__ __forceinline__ half_t tabs(half_t x) { return __builtin_fabsf16(x); }
__device__ __forceinline__ bf16_t tabs(bf16_t x) { return bf16_t(__builtin_fabsf(float(x))); }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Names of the kernels launched by the calling thread's current entry point ('+'-separated),
// for tracing tools: kernel_log_reset() at the start of an entry point, note_kernel() at every
// launch site.
void kernel_log_reset();
void note_kernel(const char *name);
const char *kernel_log();

// Workgroup size of the one-group-per-pixel kernels.  A launch of up to 2048 wavefronts runs
// one wavefront per workgroup so that it spreads over as many compute units as possible (these
// launches are bound by latency and by the load issue rate of a compute unit, not by
// occupancy); larger launches use 256 threads.
inline int group_block(int64_t threads) { return threads <= 2048 * WAVE ? WAVE : 256; }
inline int pow2_ceil(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

// ---- launch interface (one function per operator; arguments already validated) ----
hipError_t launch_sparsify(const void *in, void *prev, void *delta, int32_t *mask, float thr,
                           int32_t P, int32_t C, int dtype, hipStream_t s);
hipError_t launch_activate_truncate(void *delta, void *prev, void *trunc, int32_t *mask, float thr,
                                    int act, int mode, int32_t P, int32_t C, int dtype,
                                    hipStream_t s);
hipError_t launch_add(const void *a, const void *b, void *prev, void *out, const int32_t *ma,
                      const int32_t *mb, int32_t *mo, float wa, float wb, int act, int dense_out,
                      int32_t P, int32_t C, int dtype, hipStream_t s);
hipError_t launch_add_upsampled(const void *a, const void *b, void *prev, void *out, const int32_t *ma,
                                const int32_t *mb, int32_t *mo, float wa, float wb, int act, int32_t B,
                                int32_t H, int32_t W, int32_t C, int32_t scale, int dtype, hipStream_t s);
hipError_t launch_add_to_dense(void *a, void *b, const int32_t *ma, int act, int32_t P, int32_t C,
                               int dtype, hipStream_t s);
hipError_t launch_upsample(const void *in, void *out, const int32_t *mi, int32_t *mo, int32_t B,
                           int32_t H, int32_t W, int32_t C, int32_t scale, int dtype,
                           hipStream_t s);
hipError_t launch_concat(const void *a, const void *b, void *out, const int32_t *ma,
                         const int32_t *mb, int32_t *mo, int32_t P, int32_t Ca, int32_t Cb,
                         int dtype, hipStream_t s);
hipError_t launch_mul_add(const void *in, const int32_t *mask, void *out, int32_t *mo,
                          const void *scale, const void *bias, int32_t P, int32_t C, int dtype,
                          hipStream_t s);

struct ActEpilogue {  // optional activation/truncation fused behind a convolution
    void *prev;
    void *trunc;
    float thr;
    int act;
    int mode;
};

hipError_t launch_conv(const dc_geometry &g, const void *in, const void *filter,
                       const void *packed, const void *bias, void *out, const int32_t *mask,
                       int32_t *out_mask, int dtype, bool transposed, const ActEpilogue *epi,
                       hipStream_t s);
struct Residual {  // optional DCAdd fused behind a convolution
    const void *values;
    const int32_t *mask;
    float wa, wb;
    void *prev = nullptr;  // accumulated sum kept by a DCAdd with activation
    int act = 0;           // its activation (0: none)
};

// A layer's activation / truncation left open by its convolution and finished by the depthwise
// layer that consumes it: the layer's cached state (its truncated values receive T = truncated + v
// from the convolution), its threshold and activation.
struct OpenAct {
    void *prev = nullptr;
    void *trunc = nullptr;
    float thr = 0.f;
    int act = 0;
};
bool depthwise_closing_eligible(const dc_geometry &g, const ActEpilogue *epi, int dtype);
hipError_t launch_depthwise_closing(const dc_geometry &g, const void *in, const void *filter, void *out,
                                    const int32_t *mask, int32_t *out_mask, const ActEpilogue *epi,
                                    const OpenAct &open, int dtype, hipStream_t s);
bool pointwise_concat_eligible(const dc_geometry &g, const int32_t *channels, int n, int dtype);
hipError_t launch_pointwise_concat(const dc_geometry &g, const void *const *inputs, const int32_t *const *masks,
                                   const int32_t *channels, int n, const void *packed, void *out, int32_t *out_mask,
                                   int dtype, hipStream_t s);
bool pointwise_open_eligible(const dc_geometry &g, int dtype, int activation);
hipError_t launch_pointwise_open(const dc_geometry &g, const void *in, const void *packed, void *out,
                                 const int32_t *mask, int32_t *out_mask, const OpenAct &open, int dtype,
                                 hipStream_t s);
// Projection (+ residual sum) and the next 1x1 expansion with its activation left open, one launch.
bool pointwise_pair_eligible(const dc_geometry &gp, int expand_channels, int activation, int dtype);
hipError_t launch_pointwise_pair(const dc_geometry &gp, const void *in, const int32_t *mask,
                                 const void *project_packed, const Residual *res, void *out, int32_t *out_mask,
                                 const void *expand_packed, int expand_channels, const OpenAct &open,
                                 void *expand_out, int32_t *expand_out_mask, int dtype, hipStream_t s);
bool pointwise_eligible(const dc_geometry &g, int dtype);
bool patch_eligible(const dc_geometry &g, int dtype);
bool lds_add_eligible(const dc_geometry &g, int dtype, int activation, bool transposed = false);
hipError_t launch_lds_conv_add(const dc_geometry &g, const void *in, const void *packed, const void *bias,
                               void *out, const int32_t *mask, int32_t *out_mask, const Residual *res,
                               int dtype, hipStream_t s, bool transposed = false);
hipError_t launch_patch_conv(const dc_geometry &g, const void *in, const void *packed,
                             const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                             bool transposed, const Residual *res, int dtype, hipStream_t s,
                             const ActEpilogue *epi = nullptr, bool *epilogue_done = nullptr);
hipError_t launch_pointwise(const dc_geometry &g, const void *in, const void *packed,
                            const void *bias, void *out, const int32_t *mask, int32_t *out_mask,
                            const ActEpilogue *epi, bool *epilogue_done, const Residual *res,
                            int dtype, hipStream_t s);

// Independent small 3x3 layers launched together (dc_conv_group): each a plain convolution, a
// convolution + residual sum (res) or a convolution + activation/truncation (epi).
constexpr int CONV_GROUP_MAX = 8;
struct ConvGroupItem {
    dc_geometry g;
    const void *in;
    const int32_t *mask;
    const void *packed, *bias;
    void *out;
    int32_t *out_mask;
    const Residual *res;
    const ActEpilogue *epi;
};
bool conv_group_item_eligible(const ConvGroupItem &c, int dtype);
// the convolution kernel finishes the item's activation itself (otherwise it needs an ActGroupItem)
bool conv_group_activation_fused(const ConvGroupItem &c);
hipError_t launch_conv_group(const ConvGroupItem *items, int n, int dtype, hipStream_t s);
// ... and independent small pointwise layers (plain convolutions) likewise
bool pointwise_group_item_eligible(const ConvGroupItem &c, int dtype);
hipError_t launch_pointwise_group(const ConvGroupItem *items, int n, int dtype, hipStream_t s);

// Activation / truncation (maximum norm) of several tensors in one launch.
struct ActGroupItem {
    void *delta, *prev, *trunc;
    int32_t *mask;
    float thr;
    int32_t P, C;
};
bool act_group_eligible(const ActGroupItem *items, int n, int act, int mode, int dtype);
hipError_t launch_activate_truncate_group(const ActGroupItem *items, int n, int act, int dtype, hipStream_t s);

// Independent sums of delta tensors in one launch (dc_add_group); S > 1: the second operand is read
// through nearest upsampling from a map S times smaller.
struct AddGroupItem {
    const void *a, *b;
    void *prev, *out;
    const int32_t *ma, *mb;
    int32_t *mo;
    float wa, wb;
    int32_t act, B, H, W, C, S;
};
bool add_group_eligible(const AddGroupItem *items, int n, int dtype);
hipError_t launch_add_group(const AddGroupItem *items, int n, int dtype, hipStream_t s);
hipError_t launch_pack_filter(const dc_geometry &g, const void *filter, void *packed, int dtype,
                              bool transposed, hipStream_t s);
int64_t packed_filter_bytes(const dc_geometry &g, int dtype, bool transposed);
hipError_t launch_densify(const void *delta, void *prev, void *out, const int32_t *mask, int P, int C,
                          int dtype, hipStream_t s);
bool pool_update_eligible(const dc_geometry &g, const void *in, const void *prev, const void *out, int dtype);
hipError_t launch_pool_update(const dc_geometry &g, const void *in, void *prev, void *out, const int32_t *mask,
                              int32_t *out_mask, int dtype, hipStream_t s);
hipError_t launch_pool(const dc_geometry &g, const void *in, const void *prev, void *out,
                       const int32_t *mask, int32_t *out_mask, int mode, int dtype, bool out_f32,
                       hipStream_t s);
// Whether a 1x1-output pooling of this shape can write its result in the tensor's own type.
bool pool_global_casts(const dc_geometry &g, const void *in, const void *prev, int dtype);
hipError_t launch_pool_densify(const dc_geometry &g, const void *in, const int32_t *mask, void *acc,
                               void *dense, int dtype, hipStream_t s);
bool linear_eligible(int in_features, int dtype);
hipError_t launch_linear(const void *x, const void *w, const void *bias, void *out, int rows,
                         int in_features, int out_features, int dtype, hipStream_t s);

// Fused depthwise -> projection (-> expansion) block.  block_unsupported names the reason a
// shape is outside the kernel's range (nullptr: supported as far as the shape check goes);
// launch_block may still decline (*why != nullptr, nothing launched).
const char *block_unsupported(const dc_geometry &g, const dc_block_args &b, int dtype);
hipError_t launch_block(const dc_geometry &g, const dc_block_args &b, hipStream_t s, const char **why);
// Reduction slices (KW) the stand-alone pointwise kernel uses for this layer.
int pointwise_reduction_slices(int pixels, int in_c, int out_c);

}  // namespace dc
