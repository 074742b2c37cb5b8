// extern "C" surface of libdeltacnn_hip.so: argument validation, error reporting, dispatch.
// Every check runs before the first HIP call, so bad arguments are reported without a GPU.
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "common.hpp"

namespace {

thread_local char g_error[512] = "";
thread_local char g_kernels[256] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int finish(hipError_t e, const char *what) {
    if (e == hipSuccess) return DC_OK;
    return fail(DC_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

inline size_t esize(int dtype) { return dtype == DC_F32 ? 4 : 2; }

#define DC_REQUIRE_DTYPE(fn) \
    if (dtype != DC_F32 && dtype != DC_F16 && dtype != DC_BF16) return fail(DC_ERR_DTYPE, fn ": unsupported dtype %d", dtype)
#define DC_REQUIRE_PTR(fn, p) \
    if ((p) == nullptr) return fail(DC_ERR_NULL, fn ": " #p " is NULL")
#define DC_REQUIRE_ALIGNED(fn, p, a) \
    if ((p) != nullptr && (reinterpret_cast<uintptr_t>(p) % (a)) != 0) \
        return fail(DC_ERR_ALIGN, fn ": " #p " is not aligned to %d bytes", int(a))

// A buffer as a byte range; a NULL pointer is an empty range.
struct Span {
    uintptr_t lo, hi;
    Span(const void *p, size_t bytes) : lo(reinterpret_cast<uintptr_t>(p)), hi(p == nullptr ? 0 : reinterpret_cast<uintptr_t>(p) + bytes) {}
    bool meets(const Span &o) const { return lo < hi && o.lo < o.hi && lo < o.hi && o.lo < hi; }
};

int check_pc(const char *fn, int32_t pixels, int32_t channels) {
    if (pixels <= 0 || channels <= 0)
        return fail(DC_ERR_SHAPE, "%s: pixels=%d channels=%d must be positive", fn, pixels, channels);
    if ((int64_t)pixels * channels >= (int64_t)1 << 40)
        return fail(DC_ERR_SHAPE, "%s: tensor too large", fn);
    if (pixels > (1 << 29))
        return fail(DC_ERR_SHAPE, "%s: pixels=%d exceeds 2^29", fn, pixels);
    return DC_OK;
}

int check_geometry(const char *fn, const dc_geometry *g, bool transposed, bool pooling) {
    if (g == nullptr) return fail(DC_ERR_NULL, "%s: geometry is NULL", fn);
    if (g->batch <= 0 || g->in_h <= 0 || g->in_w <= 0 || g->in_c <= 0 || g->out_h <= 0 ||
        g->out_w <= 0 || g->out_c <= 0)
        return fail(DC_ERR_SHAPE, "%s: non-positive dimension", fn);
    if (g->in_h > 32767 || g->in_w > 32767 || g->out_h > 32767 || g->out_w > 32767 ||
        g->batch > 65535)
        return fail(DC_ERR_SHAPE, "%s: spatial dimension exceeds 32767 or batch exceeds 65535", fn);
    if ((int64_t)g->batch * g->in_h * g->in_w > (1 << 29) ||
        (int64_t)g->batch * g->out_h * g->out_w > (1 << 29))
        return fail(DC_ERR_SHAPE, "%s: more than 2^29 pixels", fn);
    if (g->kernel_h <= 0 || g->kernel_w <= 0 || g->stride_h <= 0 || g->stride_w <= 0 ||
        g->dilation_h <= 0 || g->dilation_w <= 0)
        return fail(DC_ERR_SHAPE, "%s: kernel, stride and dilation must be positive", fn);
    if (g->pad_top < 0 || g->pad_left < 0 || g->pad_bottom < 0 || g->pad_right < 0)
        return fail(DC_ERR_SHAPE, "%s: negative padding", fn);
    int eh, ew;
    if (transposed) {
        if (g->pad_top != g->pad_bottom || g->pad_left != g->pad_right)
            return fail(DC_ERR_UNSUPPORTED, "%s: transposed convolution needs symmetric padding", fn);
        eh = (g->in_h - 1) * g->stride_h - 2 * g->pad_top + g->dilation_h * (g->kernel_h - 1) + 1;
        ew = (g->in_w - 1) * g->stride_w - 2 * g->pad_left + g->dilation_w * (g->kernel_w - 1) + 1;
    } else {
        int nh = g->in_h + g->pad_top + g->pad_bottom - g->dilation_h * (g->kernel_h - 1) - 1;
        int nw = g->in_w + g->pad_left + g->pad_right - g->dilation_w * (g->kernel_w - 1) - 1;
        if (nh < 0 || nw < 0) return fail(DC_ERR_SHAPE, "%s: window larger than padded input", fn);
        eh = nh / g->stride_h + 1;
        ew = nw / g->stride_w + 1;
    }
    if (eh != g->out_h || ew != g->out_w)
        return fail(DC_ERR_SHAPE, "%s: output %dx%d does not match geometry (expected %dx%d)", fn,
                    g->out_h, g->out_w, eh, ew);
    if (pooling) {
        if (g->in_c != g->out_c) return fail(DC_ERR_SHAPE, "%s: pooling keeps the channel count", fn);
        return DC_OK;
    }
    if (g->groups <= 0 || g->in_c % g->groups != 0 || g->out_c % g->groups != 0)
        return fail(DC_ERR_SHAPE, "%s: groups=%d does not divide channels %d -> %d", fn, g->groups,
                    g->in_c, g->out_c);
    return DC_OK;
}

int check_conv(const char *fn, const dc_geometry *g, const void *input, const void *filter,
               const void *out, const int32_t *mask, const int32_t *out_mask, int dtype,
               bool transposed) {
    if (dtype != DC_F32 && dtype != DC_F16 && dtype != DC_BF16) return fail(DC_ERR_DTYPE, "%s: unsupported dtype %d", fn, dtype);
    int rc = check_geometry(fn, g, transposed, false);
    if (rc != DC_OK) return rc;
    if (!input || !filter || !out || !mask || !out_mask)
        return fail(DC_ERR_NULL, "%s: input, filter, out, mask and out_mask are required", fn);
    const bool depthwise = g->groups == g->in_c && g->groups == g->out_c;
    if (transposed && g->groups != 1)
        return fail(DC_ERR_UNSUPPORTED, "%s: transposed convolution supports groups == 1 only", fn);
    if (dtype == DC_F16 && g->groups != 1 && !depthwise)
        return fail(DC_ERR_UNSUPPORTED,
                    "%s: fp16 grouped convolution needs groups == 1 or depthwise (the reference "
                    "fp16 filter layout is only defined for those)", fn);
    size_t es = esize(dtype);
    if (reinterpret_cast<uintptr_t>(input) % es || reinterpret_cast<uintptr_t>(filter) % es ||
        reinterpret_cast<uintptr_t>(out) % es || reinterpret_cast<uintptr_t>(mask) % 4 ||
        reinterpret_cast<uintptr_t>(out_mask) % 4)
        return fail(DC_ERR_ALIGN, "%s: pointer not aligned to its element size", fn);
    return DC_OK;
}

}  // namespace

namespace dc {
void kernel_log_reset() { g_kernels[0] = 0; }
void note_kernel(const char *name) {
    const size_t used = strlen(g_kernels);
    snprintf(g_kernels + used, sizeof(g_kernels) - used, "%s%s", used ? "+" : "", name);
}
const char *kernel_log() { return g_kernels; }
}  // namespace dc

extern "C" {

const char *dc_version(void) { return "deltacnn-hip 0.1 (gfx950)"; }

const char *dc_last_error(void) { return g_error; }

const char *dc_last_kernels(void) { return g_kernels; }

int dc_sparsify(const void *input, void *prev_input, void *delta, int32_t *mask, float threshold,
                int32_t pixels, int32_t channels, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_sparsify");
    int rc = check_pc("dc_sparsify", pixels, channels);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_sparsify", input);
    DC_REQUIRE_PTR("dc_sparsify", prev_input);
    DC_REQUIRE_PTR("dc_sparsify", delta);
    DC_REQUIRE_PTR("dc_sparsify", mask);
    DC_REQUIRE_ALIGNED("dc_sparsify", input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_sparsify", prev_input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_sparsify", delta, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_sparsify", mask, 4);
    return finish(dc::launch_sparsify(input, prev_input, delta, mask, threshold, pixels, channels,
                                      dtype, (hipStream_t)stream), "dc_sparsify");
}

int dc_activate_truncate(void *delta, void *prev_input, void *truncated, int32_t *mask,
                         float threshold, int activation, int truncation_mode, int32_t pixels,
                         int32_t channels, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_activate_truncate");
    int rc = check_pc("dc_activate_truncate", pixels, channels);
    if (rc != DC_OK) return rc;
    if (activation > DC_ACT_SWISH)
        return fail(DC_ERR_UNSUPPORTED, "dc_activate_truncate: activation id %d", activation);
    if (truncation_mode > DC_TRUNC_RMS)
        return fail(DC_ERR_UNSUPPORTED, "dc_activate_truncate: truncation mode %d", truncation_mode);
    DC_REQUIRE_PTR("dc_activate_truncate", delta);
    DC_REQUIRE_PTR("dc_activate_truncate", prev_input);
    DC_REQUIRE_PTR("dc_activate_truncate", mask);
    if (truncation_mode >= 0) DC_REQUIRE_PTR("dc_activate_truncate", truncated);
    DC_REQUIRE_ALIGNED("dc_activate_truncate", delta, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_activate_truncate", prev_input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_activate_truncate", truncated, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_activate_truncate", mask, 4);
    return finish(dc::launch_activate_truncate(delta, prev_input, truncated, mask, threshold,
                                               activation, truncation_mode, pixels, channels,
                                               dtype, (hipStream_t)stream), "dc_activate_truncate");
}

int dc_conv(const dc_geometry *g, const void *input, const void *filter, const void *packed_filter,
            const void *bias, void *out, const int32_t *mask, int32_t *out_mask, int dtype,
            void *stream) {
    dc::kernel_log_reset();
    int rc = check_conv("dc_conv", g, input, filter, out, mask, out_mask, dtype, false);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_ALIGNED("dc_conv", packed_filter, 16);
    return finish(dc::launch_conv(*g, input, filter, packed_filter, bias, out, mask, out_mask,
                                  dtype, false, nullptr, (hipStream_t)stream), "dc_conv");
}

int dc_conv_act(const dc_geometry *g, const void *input, const void *filter,
                const void *packed_filter, const void *bias, void *out, const int32_t *mask,
                int32_t *out_mask, void *prev_out, void *truncated, float threshold, int activation,
                int truncation_mode, int dtype, void *stream) {
    dc::kernel_log_reset();
    int rc = check_conv("dc_conv_act", g, input, filter, out, mask, out_mask, dtype, false);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_ALIGNED("dc_conv_act", packed_filter, 16);
    DC_REQUIRE_PTR("dc_conv_act", prev_out);
    if (truncation_mode >= 0) DC_REQUIRE_PTR("dc_conv_act", truncated);
    if (activation > DC_ACT_SWISH || truncation_mode > DC_TRUNC_RMS)
        return fail(DC_ERR_UNSUPPORTED, "dc_conv_act: activation %d / truncation mode %d",
                    activation, truncation_mode);
    dc::ActEpilogue epi{prev_out, truncated, threshold, activation, truncation_mode};
    return finish(dc::launch_conv(*g, input, filter, packed_filter, bias, out, mask, out_mask,
                                  dtype, false, &epi, (hipStream_t)stream), "dc_conv_act");
}

int dc_conv_add(const dc_geometry *g, const void *input, const void *packed_filter,
                const void *bias, const int32_t *mask, const void *residual,
                const int32_t *mask_residual, void *out, int32_t *out_mask, float weight_residual,
                float weight_conv, void *prev_out, int activation, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_conv_add");
    int rc = check_geometry("dc_conv_add", g, false, false);
    if (rc != DC_OK) return rc;
    if (activation < 0 || activation > DC_ACT_SWISH)
        return fail(DC_ERR_UNSUPPORTED, "dc_conv_add: activation %d", activation);
    const bool pointwise = dc::pointwise_eligible(*g, dtype);
    const bool patch = !pointwise && dc::patch_eligible(*g, dtype);
    if (!pointwise && !patch && !dc::lds_add_eligible(*g, dtype, activation))
        return fail(DC_ERR_UNSUPPORTED, "dc_conv_add: only 16-bit 1x1 stride-1 convolutions with "
                                        "Cin %% 8 == 0 and Cout %% 4 == 0 and 16-bit K x K layers "
                                        "with Cin %% 8 == 0 and at most 64 taps have the fused form");
    DC_REQUIRE_PTR("dc_conv_add", input);
    DC_REQUIRE_PTR("dc_conv_add", packed_filter);
    DC_REQUIRE_PTR("dc_conv_add", mask);
    DC_REQUIRE_PTR("dc_conv_add", residual);
    DC_REQUIRE_PTR("dc_conv_add", mask_residual);
    DC_REQUIRE_PTR("dc_conv_add", out);
    DC_REQUIRE_PTR("dc_conv_add", out_mask);
    if (activation > 0) DC_REQUIRE_PTR("dc_conv_add", prev_out);
    DC_REQUIRE_ALIGNED("dc_conv_add", input, 16);
    DC_REQUIRE_ALIGNED("dc_conv_add", packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_conv_add", residual, 8);
    DC_REQUIRE_ALIGNED("dc_conv_add", out, 8);
    DC_REQUIRE_ALIGNED("dc_conv_add", prev_out, 8);
    DC_REQUIRE_ALIGNED("dc_conv_add", bias, 8);
    dc::Residual res{residual, mask_residual, weight_residual, weight_conv, prev_out, activation};
    if (pointwise) {
        bool unused = false;
        return finish(dc::launch_pointwise(*g, input, packed_filter, bias, out, mask, out_mask, nullptr,
                                           &unused, &res, dtype, (hipStream_t)stream), "dc_conv_add");
    }
    if (!patch)
        return finish(dc::launch_lds_conv_add(*g, input, packed_filter, bias, out, mask, out_mask, &res, dtype,
                                              (hipStream_t)stream), "dc_conv_add");
    return finish(dc::launch_patch_conv(*g, input, packed_filter, bias, out, mask, out_mask, false, &res,
                                        dtype, (hipStream_t)stream), "dc_conv_add");
}

int64_t dc_packed_filter_bytes(const dc_geometry *g, int dtype, int transposed) {
    if (g == nullptr || g->in_c <= 0 || g->out_c <= 0 || g->kernel_h <= 0 || g->kernel_w <= 0 ||
        g->groups <= 0)
        return 0;
    return dc::packed_filter_bytes(*g, dtype, transposed != 0);
}

int dc_pack_filter(const dc_geometry *g, const void *filter, void *packed_filter, int dtype,
                   int transposed, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_pack_filter");
    if (g == nullptr) return fail(DC_ERR_NULL, "dc_pack_filter: geometry is NULL");
    if (dc_packed_filter_bytes(g, dtype, transposed) == 0)
        return fail(DC_ERR_UNSUPPORTED, "dc_pack_filter: this convolution has no packed form");
    DC_REQUIRE_PTR("dc_pack_filter", filter);
    DC_REQUIRE_PTR("dc_pack_filter", packed_filter);
    DC_REQUIRE_ALIGNED("dc_pack_filter", filter, 2);
    DC_REQUIRE_ALIGNED("dc_pack_filter", packed_filter, 16);
    return finish(dc::launch_pack_filter(*g, filter, packed_filter, dtype, transposed != 0,
                                         (hipStream_t)stream), "dc_pack_filter");
}

int dc_deconv(const dc_geometry *g, const void *input, const void *filter,
              const void *packed_filter, const void *bias, void *out, const int32_t *mask,
              int32_t *out_mask, int dtype, void *stream) {
    dc::kernel_log_reset();
    int rc = check_conv("dc_deconv", g, input, filter, out, mask, out_mask, dtype, true);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_ALIGNED("dc_deconv", packed_filter, 16);
    return finish(dc::launch_conv(*g, input, filter, packed_filter, bias, out, mask, out_mask,
                                  dtype, true, nullptr, (hipStream_t)stream), "dc_deconv");
}

int dc_deconv_add(const dc_geometry *g, const void *input, const void *packed_filter, const int32_t *mask,
                  const void *residual, const int32_t *mask_residual, void *out, int32_t *out_mask,
                  float weight_residual, float weight_conv, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_deconv_add");
    int rc = check_geometry("dc_deconv_add", g, true, false);
    if (rc != DC_OK) return rc;
    if (!dc::lds_add_eligible(*g, dtype, 0, true))
        return fail(DC_ERR_UNSUPPORTED, "dc_deconv_add: only 16-bit transposed convolutions of the LDS-halo kernel "
                                        "(Cin %% 8 == 0, groups 1, dilation 1, window >= stride, too large for the "
                                        "4x4-patch kernel) have the fused form");
    DC_REQUIRE_PTR("dc_deconv_add", input);
    DC_REQUIRE_PTR("dc_deconv_add", packed_filter);
    DC_REQUIRE_PTR("dc_deconv_add", mask);
    DC_REQUIRE_PTR("dc_deconv_add", residual);
    DC_REQUIRE_PTR("dc_deconv_add", mask_residual);
    DC_REQUIRE_PTR("dc_deconv_add", out);
    DC_REQUIRE_PTR("dc_deconv_add", out_mask);
    DC_REQUIRE_ALIGNED("dc_deconv_add", input, 16);
    DC_REQUIRE_ALIGNED("dc_deconv_add", packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_deconv_add", residual, 8);
    DC_REQUIRE_ALIGNED("dc_deconv_add", out, 8);
    {
        // every output tile reads the residual of its pixels and other tiles' workgroups may have
        // stored theirs by then: the sum is not taken in place
        const size_t po = (size_t)g->batch * g->out_h * g->out_w, es = esize(dtype);
        const Span o(out, po * g->out_c * es), om(out_mask, po * 4);
        const Span rd[] = {Span(residual, po * g->out_c * es), Span(mask_residual, po * 4),
                           Span(input, (size_t)g->batch * g->in_h * g->in_w * g->in_c * es),
                           Span(mask, (size_t)g->batch * g->in_h * g->in_w * 4)};
        for (const Span &r : rd)
            if (o.meets(r) || om.meets(r))
                return fail(DC_ERR_UNSUPPORTED, "dc_deconv_add: out / out_mask overlap an input of the call");
    }
    dc::Residual res{residual, mask_residual, weight_residual, weight_conv, nullptr, 0};
    return finish(dc::launch_lds_conv_add(*g, input, packed_filter, nullptr, out, mask, out_mask, &res, dtype,
                                          (hipStream_t)stream, true), "dc_deconv_add");
}

int dc_pool(const dc_geometry *g, const void *input, const void *prev_input, void *out,
            const int32_t *mask, int32_t *out_mask, int pooling_mode, int dtype,
            int global_out_dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_pool");
    int rc = check_geometry("dc_pool", g, false, true);
    if (rc != DC_OK) return rc;
    if (pooling_mode != DC_POOL_MAX && pooling_mode != DC_POOL_AVG)
        return fail(DC_ERR_UNSUPPORTED, "dc_pool: pooling mode %d", pooling_mode);
    DC_REQUIRE_PTR("dc_pool", input);
    DC_REQUIRE_PTR("dc_pool", out);
    DC_REQUIRE_PTR("dc_pool", mask);
    DC_REQUIRE_PTR("dc_pool", out_mask);
    if (pooling_mode == DC_POOL_MAX) DC_REQUIRE_PTR("dc_pool", prev_input);
    DC_REQUIRE_ALIGNED("dc_pool", input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_pool", prev_input, esize(dtype));
    const bool global = g->out_h == 1 && g->out_w == 1;
    bool out_f32 = true;
    if (global) {
        if (global_out_dtype != DC_F32 && global_out_dtype != dtype)
            return fail(DC_ERR_DTYPE, "dc_pool: global_out_dtype %d is neither float32 nor the tensor type",
                        global_out_dtype);
        out_f32 = global_out_dtype == DC_F32;
        if (!out_f32 && !dc::pool_global_casts(*g, input, prev_input, dtype))
            return fail(DC_ERR_UNSUPPORTED, "dc_pool: this shape needs a float32 output buffer");
    }
    DC_REQUIRE_ALIGNED("dc_pool", out, (global && out_f32) ? 4 : esize(dtype));
    return finish(dc::launch_pool(*g, input, prev_input, out, mask, out_mask, pooling_mode, dtype,
                                  out_f32, (hipStream_t)stream), "dc_pool");
}

int dc_concat_conv(const dc_geometry *g, int32_t count, const void *const *inputs, const int32_t *const *masks,
                   const int32_t *channels, const void *packed_filter, void *out, int32_t *out_mask, int dtype,
                   void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_concat_conv");
    int rc = check_geometry("dc_concat_conv", g, false, false);
    if (rc != DC_OK) return rc;
    if (count < 2 || count > 4)
        return fail(DC_ERR_SHAPE, "dc_concat_conv: count=%d outside 2..4", count);
    DC_REQUIRE_PTR("dc_concat_conv", inputs);
    DC_REQUIRE_PTR("dc_concat_conv", masks);
    DC_REQUIRE_PTR("dc_concat_conv", channels);
    if (!dc::pointwise_concat_eligible(*g, channels, count, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_concat_conv: needs a 16-bit 1x1 stride-1 convolution without padding "
                                        "(Cout %% 4 == 0) over tensors with channels in multiples of 32 that add up "
                                        "to in_c");
    DC_REQUIRE_PTR("dc_concat_conv", packed_filter);
    DC_REQUIRE_PTR("dc_concat_conv", out);
    DC_REQUIRE_PTR("dc_concat_conv", out_mask);
    DC_REQUIRE_ALIGNED("dc_concat_conv", packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_concat_conv", out, 8);
    const size_t P = (size_t)g->batch * g->in_h * g->in_w, es = esize(dtype);
    const Span o(out, P * g->out_c * es), om(out_mask, P * 4);
    for (int i = 0; i < count; ++i) {
        if (inputs[i] == nullptr || masks[i] == nullptr)
            return fail(DC_ERR_NULL, "dc_concat_conv: input %d or its mask is NULL", i);
        if (reinterpret_cast<uintptr_t>(inputs[i]) % 16 != 0)
            return fail(DC_ERR_ALIGN, "dc_concat_conv: input %d is not aligned to 16 bytes", i);
        const Span in(inputs[i], P * channels[i] * es), im(masks[i], P * 4);
        if (o.meets(in) || o.meets(im) || om.meets(in) || om.meets(im))
            return fail(DC_ERR_UNSUPPORTED, "dc_concat_conv: out / out_mask overlap input %d", i);
    }
    return finish(dc::launch_pointwise_concat(*g, inputs, masks, channels, count, packed_filter, out, out_mask, dtype,
                                              (hipStream_t)stream), "dc_concat_conv");
}

int dc_pool_update(const dc_geometry *g, const void *input, void *prev_input, void *out, const int32_t *mask,
                   int32_t *out_mask, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_pool_update");
    int rc = check_geometry("dc_pool_update", g, false, true);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_pool_update", input);
    DC_REQUIRE_PTR("dc_pool_update", prev_input);
    DC_REQUIRE_PTR("dc_pool_update", out);
    DC_REQUIRE_PTR("dc_pool_update", mask);
    DC_REQUIRE_PTR("dc_pool_update", out_mask);
    if (!dc::pool_update_eligible(*g, input, prev_input, out, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_pool_update: needs 2x2 or 3x3 windows that tile the map exactly (window == "
                                        "stride, no padding, no dilation, input = output * stride), channels in whole "
                                        "16-byte vectors, 16-byte aligned tensors and at most 2^20 lanes");
    {
        const size_t pi = (size_t)g->batch * g->in_h * g->in_w, po = (size_t)g->batch * g->out_h * g->out_w, es = esize(dtype);
        const Span wr[] = {Span(prev_input, pi * g->in_c * es), Span(out, po * g->in_c * es), Span(out_mask, po * 4)};
        const Span rd[] = {Span(input, pi * g->in_c * es), Span(mask, pi * 4)};
        for (size_t i = 0; i < 3; ++i) {
            for (const Span &r : rd)
                if (wr[i].meets(r)) return fail(DC_ERR_UNSUPPORTED, "dc_pool_update: an output overlaps an input of the call");
            for (size_t j = i + 1; j < 3; ++j)
                if (wr[i].meets(wr[j])) return fail(DC_ERR_UNSUPPORTED, "dc_pool_update: two outputs of the call overlap");
        }
    }
    return finish(dc::launch_pool_update(*g, input, prev_input, out, mask, out_mask, dtype, (hipStream_t)stream),
                  "dc_pool_update");
}

int dc_add(const void *a, const void *b, void *prev_out, void *out, const int32_t *mask_a,
           const int32_t *mask_b, int32_t *mask_out, float weight_a, float weight_b, int activation,
           int dense_out, int32_t pixels, int32_t channels, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_add");
    int rc = check_pc("dc_add", pixels, channels);
    if (rc != DC_OK) return rc;
    if (activation > DC_ACT_SWISH) return fail(DC_ERR_UNSUPPORTED, "dc_add: activation id %d", activation);
    DC_REQUIRE_PTR("dc_add", a);
    DC_REQUIRE_PTR("dc_add", b);
    DC_REQUIRE_PTR("dc_add", out);
    DC_REQUIRE_PTR("dc_add", mask_a);
    DC_REQUIRE_PTR("dc_add", mask_b);
    if (!dense_out) DC_REQUIRE_PTR("dc_add", mask_out);
    if (dense_out || activation > 0) DC_REQUIRE_PTR("dc_add", prev_out);
    DC_REQUIRE_ALIGNED("dc_add", a, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add", b, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add", out, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add", prev_out, esize(dtype));
    return finish(dc::launch_add(a, b, prev_out, out, mask_a, mask_b, mask_out, weight_a, weight_b,
                                 activation, dense_out, pixels, channels, dtype,
                                 (hipStream_t)stream), "dc_add");
}

int dc_add_upsampled(const void *a, const void *b, void *prev_out, void *out, const int32_t *mask_a,
                     const int32_t *mask_b, int32_t *mask_out, float weight_a, float weight_b,
                     int activation, int32_t batch, int32_t height, int32_t width, int32_t channels,
                     int32_t scale, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_add_upsampled");
    if (batch <= 0 || height <= 0 || width <= 0 || scale <= 0)
        return fail(DC_ERR_SHAPE, "dc_add_upsampled: batch, height, width and scale must be positive");
    if (height % scale != 0 || width % scale != 0)
        return fail(DC_ERR_SHAPE, "dc_add_upsampled: %d x %d is not a multiple of scale %d", height, width, scale);
    if ((int64_t)batch * height * width > INT32_MAX)
        return fail(DC_ERR_SHAPE, "dc_add_upsampled: more than 2^31 pixels");
    int rc = check_pc("dc_add_upsampled", batch * height * width, channels);
    if (rc != DC_OK) return rc;
    if (activation > DC_ACT_SWISH) return fail(DC_ERR_UNSUPPORTED, "dc_add_upsampled: activation id %d", activation);
    DC_REQUIRE_PTR("dc_add_upsampled", a);
    DC_REQUIRE_PTR("dc_add_upsampled", b);
    DC_REQUIRE_PTR("dc_add_upsampled", out);
    DC_REQUIRE_PTR("dc_add_upsampled", mask_a);
    DC_REQUIRE_PTR("dc_add_upsampled", mask_b);
    DC_REQUIRE_PTR("dc_add_upsampled", mask_out);
    if (activation > 0) DC_REQUIRE_PTR("dc_add_upsampled", prev_out);
    DC_REQUIRE_ALIGNED("dc_add_upsampled", a, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add_upsampled", b, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add_upsampled", out, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add_upsampled", prev_out, esize(dtype));
    return finish(dc::launch_add_upsampled(a, b, prev_out, out, mask_a, mask_b, mask_out, weight_a, weight_b,
                                           activation, batch, height, width, channels, scale, dtype,
                                           (hipStream_t)stream), "dc_add_upsampled");
}

int dc_densify(const void *delta, void *prev_out, void *out, const int32_t *mask, int32_t pixels,
               int32_t channels, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_densify");
    int rc = check_pc("dc_densify", pixels, channels);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_densify", delta);
    DC_REQUIRE_PTR("dc_densify", prev_out);
    DC_REQUIRE_PTR("dc_densify", out);
    DC_REQUIRE_PTR("dc_densify", mask);
    DC_REQUIRE_ALIGNED("dc_densify", delta, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_densify", prev_out, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_densify", out, esize(dtype));
    return finish(dc::launch_densify(delta, prev_out, out, mask, pixels, channels, dtype,
                                     (hipStream_t)stream), "dc_densify");
}

int dc_expand_depthwise(const dc_geometry *g, const dc_expand_dw_args *args, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_expand_depthwise");
    int rc = check_geometry("dc_expand_depthwise", g, false, false);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_expand_depthwise", args);
    const dc_expand_dw_args &a = *args;
    if (dtype != DC_F16 && dtype != DC_BF16)
        return fail(DC_ERR_UNSUPPORTED, "dc_expand_depthwise: 16-bit types only");
    if (a.expand_in_channels <= 0)
        return fail(DC_ERR_SHAPE, "dc_expand_depthwise: expand_in_channels=%d must be positive", a.expand_in_channels);
    if (a.expand_activation > DC_ACT_SWISH || a.dw_activation > DC_ACT_SWISH || a.dw_truncation_mode > DC_TRUNC_RMS)
        return fail(DC_ERR_UNSUPPORTED, "dc_expand_depthwise: activation or truncation mode out of range");
    if (a.expand_truncation_mode != DC_TRUNC_MAX)
        return fail(DC_ERR_UNSUPPORTED, "dc_expand_depthwise: the expansion's truncation has to be the maximum norm");
    // the expansion as a 1x1 convolution on the depthwise layer's input map
    dc_geometry ge = *g;
    ge.in_c = a.expand_in_channels;
    ge.out_h = g->in_h; ge.out_w = g->in_w; ge.out_c = g->in_c;
    ge.kernel_h = ge.kernel_w = 1;
    ge.stride_h = ge.stride_w = ge.dilation_h = ge.dilation_w = 1;
    ge.pad_top = ge.pad_left = ge.pad_bottom = ge.pad_right = 0;
    ge.groups = 1;
    const bool opened = a.expand_packed_filter == nullptr;  // dc_project_expand ran the convolution
    if (!opened && !dc::pointwise_open_eligible(ge, dtype, a.expand_activation))
        return fail(DC_ERR_UNSUPPORTED, "dc_expand_depthwise: the expansion needs input channels in multiples of 8, "
                                        "output channels in multiples of 8 and ReLU or ReLU6");
    dc::ActEpilogue dw_epi{a.dw_prev_out, a.dw_truncated, a.dw_threshold, a.dw_activation, a.dw_truncation_mode};
    if (!dc::depthwise_closing_eligible(*g, &dw_epi, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_expand_depthwise: needs a depthwise 3x3 convolution with stride 1 or 2 and "
                                        "padding 1 on a map small enough for the per-pixel kernel (input of at "
                                        "most 2 MB, at most two 16-byte vectors per lane, one with stride 2) with a "
                                        "truncating activation");
    if (!opened) {
        DC_REQUIRE_PTR("dc_expand_depthwise", a.input);
        DC_REQUIRE_PTR("dc_expand_depthwise", a.mask);
        DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.input, 16);
        DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.expand_packed_filter, 16);
    }
    DC_REQUIRE_PTR("dc_expand_depthwise", a.expand_prev_out);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.expand_truncated);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.expand_out);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.expand_out_mask);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.dw_filter);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.dw_prev_out);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.dw_truncated);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.out);
    DC_REQUIRE_PTR("dc_expand_depthwise", a.out_mask);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.expand_prev_out, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.expand_truncated, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.expand_out, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.dw_filter, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.dw_prev_out, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.dw_truncated, 16);
    DC_REQUIRE_ALIGNED("dc_expand_depthwise", a.out, 16);
    dc::OpenAct open;
    open.prev = a.expand_prev_out;
    open.trunc = a.expand_truncated;
    open.thr = a.expand_threshold;
    open.act = a.expand_activation;
    if (!opened) {
        hipError_t e = dc::launch_pointwise_open(ge, a.input, a.expand_packed_filter, a.expand_out, a.mask,
                                                 a.expand_out_mask, open, dtype, (hipStream_t)stream);
        if (e != hipSuccess) return finish(e, "dc_expand_depthwise");
    }
    return finish(dc::launch_depthwise_closing(*g, a.expand_out, a.dw_filter, a.out, a.expand_out_mask, a.out_mask,
                                               &dw_epi, open, dtype, (hipStream_t)stream),
                  "dc_expand_depthwise");
}

int dc_project_expand(const dc_geometry *g, const dc_project_expand_args *args, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_project_expand");
    int rc = check_geometry("dc_project_expand", g, false, false);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_project_expand", args);
    const dc_project_expand_args &a = *args;
    if (dtype != DC_F16 && dtype != DC_BF16)
        return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: 16-bit types only");
    if (a.expand_channels <= 0)
        return fail(DC_ERR_SHAPE, "dc_project_expand: expand_channels=%d must be positive", a.expand_channels);
    if (a.expand_activation > DC_ACT_SWISH || a.dw_activation > DC_ACT_SWISH || a.dw_truncation_mode > DC_TRUNC_RMS)
        return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: activation or truncation mode out of range");
    if (!dc::pointwise_pair_eligible(*g, a.expand_channels, a.expand_activation, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: needs 1x1 layers with block output channels in multiples "
                                        "of 32 up to 96, a projection filter of at most 128 KB, ReLU or ReLU6 and a "
                                        "map small enough for the reduction-slice form of the projection");
    DC_REQUIRE_PTR("dc_project_expand", a.dw_geometry);
    rc = check_geometry("dc_project_expand", a.dw_geometry, false, false);
    if (rc != DC_OK) return rc;
    const dc_geometry &gd = *a.dw_geometry;
    if (gd.batch != g->batch || gd.in_h != g->out_h || gd.in_w != g->out_w || gd.in_c != a.expand_channels)
        return fail(DC_ERR_SHAPE, "dc_project_expand: dw_geometry does not describe a layer on the expansion's output");
    DC_REQUIRE_PTR("dc_project_expand", a.input);
    DC_REQUIRE_PTR("dc_project_expand", a.mask);
    DC_REQUIRE_PTR("dc_project_expand", a.project_packed_filter);
    DC_REQUIRE_PTR("dc_project_expand", a.out);
    DC_REQUIRE_PTR("dc_project_expand", a.out_mask);
    if (a.residual != nullptr) DC_REQUIRE_PTR("dc_project_expand", a.residual_mask);
    DC_REQUIRE_PTR("dc_project_expand", a.expand_packed_filter);
    DC_REQUIRE_PTR("dc_project_expand", a.expand_prev_out);
    DC_REQUIRE_PTR("dc_project_expand", a.expand_truncated);
    DC_REQUIRE_PTR("dc_project_expand", a.expand_out);
    DC_REQUIRE_PTR("dc_project_expand", a.expand_out_mask);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.input, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.project_packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.residual, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.out, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.expand_packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.expand_prev_out, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.expand_truncated, 16);
    DC_REQUIRE_ALIGNED("dc_project_expand", a.expand_out, 16);
    {
        // the state pointers do not enter the decision; placeholders that pass its alignment tests
        dc::ActEpilogue probe{a.expand_prev_out, a.expand_truncated, 0.f, a.dw_activation, a.dw_truncation_mode};
        if (!dc::depthwise_closing_eligible(gd, &probe, dtype))
            return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: the depthwise layer behind the expansion cannot finish "
                                            "its activation (needs 3x3, stride 1 or 2, padding 1 on a small map)");
    }
    {
        // Several workgroups per pixel tile read every input of this call and repeat the projection
        // while one of them stores it: nothing the call writes may overlap anything it reads or
        // anything else it writes (expand_truncated is read and written by the same lanes).
        const size_t P = (size_t)g->batch * g->out_h * g->out_w, es = esize(dtype);
        const Span wr[] = {Span(a.out, P * g->out_c * es), Span(a.out_mask, P * 4), Span(a.expand_out_mask, P * 4),
                           Span(a.expand_out, P * a.expand_channels * es), Span(a.expand_truncated, P * a.expand_channels * es)};
        const Span rd[] = {Span(a.input, P * g->in_c * es), Span(a.mask, P * 4), Span(a.residual, P * g->out_c * es),
                           Span(a.residual_mask, P * 4), Span(a.expand_prev_out, P * a.expand_channels * es),
                           Span(a.project_packed_filter, (size_t)dc_packed_filter_bytes(g, dtype, 0)),
                           Span(a.expand_packed_filter, (size_t)((g->out_c + 31) / 32 * 32) * ((a.expand_channels + 15) / 16 * 16) * es)};
        for (size_t i = 0; i < sizeof(wr) / sizeof(wr[0]); ++i) {
            for (size_t j = 0; j < sizeof(rd) / sizeof(rd[0]); ++j)
                if (wr[i].meets(rd[j]))
                    return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: an output buffer overlaps an input of the call "
                                                    "(no in-place sums: out, out_mask, expand_out, expand_out_mask and "
                                                    "expand_truncated must be separate from input, mask, residual, "
                                                    "residual_mask, expand_prev_out and the filters)");
            for (size_t j = i + 1; j < sizeof(wr) / sizeof(wr[0]); ++j)
                if (wr[i].meets(wr[j]))
                    return fail(DC_ERR_UNSUPPORTED, "dc_project_expand: two output buffers of the call overlap");
        }
    }
    dc::Residual res{a.residual, a.residual_mask, a.weight_residual, a.weight_conv};
    dc::OpenAct open;
    open.prev = a.expand_prev_out;
    open.trunc = a.expand_truncated;
    open.act = a.expand_activation;
    return finish(dc::launch_pointwise_pair(*g, a.input, a.mask, a.project_packed_filter,
                                            a.residual != nullptr ? &res : nullptr, a.out, a.out_mask,
                                            a.expand_packed_filter, a.expand_channels, open, a.expand_out,
                                            a.expand_out_mask, dtype, (hipStream_t)stream),
                  "dc_project_expand");
}

int dc_conv_group(const dc_conv_item *items, int32_t count, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_conv_group");
    DC_REQUIRE_PTR("dc_conv_group", items);
    if (count < 2 || count > DC_CONV_GROUP_MAX)
        return fail(DC_ERR_SHAPE, "dc_conv_group: count=%d outside 2..%d", count, int(DC_CONV_GROUP_MAX));
    dc::ConvGroupItem conv[DC_CONV_GROUP_MAX];
    dc::Residual res[DC_CONV_GROUP_MAX];
    dc::ActEpilogue epi[DC_CONV_GROUP_MAX];
    dc::ActGroupItem act[DC_CONV_GROUP_MAX];
    int n_act = 0, act_kind = 0;
    bool pointwise = false;
    for (int i = 0; i < count; ++i) {
        const dc_conv_item &it = items[i];
        int rc = check_conv("dc_conv_group", &it.geometry, it.input, it.packed_filter, it.out, it.mask, it.out_mask,
                            dtype, false);
        if (rc != DC_OK) return rc;
        DC_REQUIRE_ALIGNED("dc_conv_group", it.input, 16);
        DC_REQUIRE_ALIGNED("dc_conv_group", it.packed_filter, 16);
        DC_REQUIRE_ALIGNED("dc_conv_group", it.out, 8);
        DC_REQUIRE_ALIGNED("dc_conv_group", it.bias, 8);
        const dc_geometry &g = it.geometry;
        conv[i] = dc::ConvGroupItem{g, it.input, it.mask, it.packed_filter, it.bias, it.out, it.out_mask, nullptr, nullptr};
        if (it.residual != nullptr) {
            if (it.prev_out != nullptr)
                return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: item %d has a residual sum and an activation", i);
            if (it.sum_activation < 0 || it.sum_activation > DC_ACT_SWISH)
                return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: item %d: activation %d", i, it.sum_activation);
            DC_REQUIRE_PTR("dc_conv_group", it.residual_mask);
            if (it.sum_activation > 0) DC_REQUIRE_PTR("dc_conv_group", it.sum_prev_out);
            DC_REQUIRE_ALIGNED("dc_conv_group", it.residual, 8);
            DC_REQUIRE_ALIGNED("dc_conv_group", it.sum_prev_out, 8);
            res[i] = dc::Residual{it.residual, it.residual_mask, it.weight_residual, it.weight_conv, it.sum_prev_out,
                                  it.sum_activation};
            conv[i].res = &res[i];
        } else if (it.prev_out != nullptr) {
            DC_REQUIRE_PTR("dc_conv_group", it.truncated);
            if (it.activation > DC_ACT_SWISH || it.truncation_mode != DC_TRUNC_MAX)
                return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: item %d: activation %d / truncation mode %d", i,
                            it.activation, it.truncation_mode);
            epi[i] = dc::ActEpilogue{it.prev_out, it.truncated, it.threshold, it.activation, it.truncation_mode};
            conv[i].epi = &epi[i];
        }
        const bool pw = dc::pointwise_group_item_eligible(conv[i], dtype);
        if (!pw && !dc::conv_group_item_eligible(conv[i], dtype))
            return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: item %d is neither a 16-bit 3x3 layer of the 4x4-patch kernel "
                                            "(Cin %% 8 == 0, patches * channel tiles * steps <= 32768) nor a plain 1x1 "
                                            "convolution of the one-tile pointwise arrangement", i);
        if (i > 0 && pw != pointwise)
            return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: 1x1 and 3x3 layers in one group");
        pointwise = pw;
        if (conv[i].epi != nullptr && !dc::conv_group_activation_fused(conv[i])) {
            const int kind = it.activation < 0 ? 0 : it.activation;
            if (n_act > 0 && kind != act_kind)
                return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: activations %d and %d in one group", act_kind, kind);
            act_kind = kind;
            act[n_act++] = dc::ActGroupItem{it.out, it.prev_out, it.truncated, it.out_mask, it.threshold,
                                            g.batch * g.out_h * g.out_w, g.out_c};
        }
    }
    // All items run side by side in one launch: no item may write bytes that another reads or
    // writes (byte ranges, so views into one allocation are seen too).
    for (int i = 0; i < count; ++i)
        for (int j = 0; j < count; ++j) {
            if (i == j) continue;
            const dc_conv_item &a = items[i], &b = items[j];
            const size_t es = esize(dtype);
            const size_t pa = (size_t)a.geometry.batch * a.geometry.out_h * a.geometry.out_w, ca = a.geometry.out_c;
            const size_t pb = (size_t)b.geometry.batch * b.geometry.out_h * b.geometry.out_w, cb = b.geometry.out_c;
            const size_t pbi = (size_t)b.geometry.batch * b.geometry.in_h * b.geometry.in_w;
            const Span wr[] = {Span(a.out, pa * ca * es), Span(a.out_mask, pa * 4), Span(a.prev_out, pa * ca * es),
                               Span(a.truncated, pa * ca * es), Span(a.sum_prev_out, pa * ca * es)};
            const Span other[] = {Span(b.input, pbi * b.geometry.in_c * es), Span(b.mask, pbi * 4),
                                  Span(b.residual, pb * cb * es), Span(b.residual_mask, pb * 4), Span(b.bias, cb * es),
                                  Span(b.out, pb * cb * es), Span(b.out_mask, pb * 4), Span(b.prev_out, pb * cb * es),
                                  Span(b.truncated, pb * cb * es), Span(b.sum_prev_out, pb * cb * es)};
            for (const Span &w : wr)
                for (const Span &o : other)
                    if (w.meets(o))
                        return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: items %d and %d share a buffer one of them writes", i, j);
        }
    if (n_act > 1 && !dc::act_group_eligible(act, n_act, act_kind, DC_TRUNC_MAX, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_conv_group: an activation outside the grouped kernel's range "
                                        "(out_c %% 8 == 0, out_c <= 2048, tensor <= 1 MB, 16-byte aligned)");
    if (pointwise)
        return finish(dc::launch_pointwise_group(conv, count, dtype, (hipStream_t)stream), "dc_conv_group");
    hipError_t e = dc::launch_conv_group(conv, count, dtype, (hipStream_t)stream);
    if (e == hipSuccess && n_act == 1)
        e = dc::launch_activate_truncate(act[0].delta, act[0].prev, act[0].trunc, act[0].mask, act[0].thr, act_kind,
                                         DC_TRUNC_MAX, act[0].P, act[0].C, dtype, (hipStream_t)stream);
    else if (e == hipSuccess && n_act > 1)
        e = dc::launch_activate_truncate_group(act, n_act, act_kind, dtype, (hipStream_t)stream);
    return finish(e, "dc_conv_group");
}

int dc_add_group(const dc_add_item *items, int32_t count, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_add_group");
    DC_REQUIRE_PTR("dc_add_group", items);
    if (count < 2 || count > DC_CONV_GROUP_MAX)
        return fail(DC_ERR_SHAPE, "dc_add_group: count=%d outside 2..%d", count, int(DC_CONV_GROUP_MAX));
    dc::AddGroupItem sums[DC_CONV_GROUP_MAX];
    for (int i = 0; i < count; ++i) {
        const dc_add_item &it = items[i];
        if (it.batch <= 0 || it.height <= 0 || it.width <= 0 || it.scale <= 0)
            return fail(DC_ERR_SHAPE, "dc_add_group: item %d: batch, height, width and scale must be positive", i);
        if (it.height % it.scale != 0 || it.width % it.scale != 0)
            return fail(DC_ERR_SHAPE, "dc_add_group: item %d: %d x %d is not a multiple of scale %d", i, it.height,
                        it.width, it.scale);
        if ((int64_t)it.batch * it.height * it.width > INT32_MAX)
            return fail(DC_ERR_SHAPE, "dc_add_group: item %d: more than 2^31 pixels", i);
        int rc = check_pc("dc_add_group", it.batch * it.height * it.width, it.channels);
        if (rc != DC_OK) return rc;
        if (it.activation > DC_ACT_SWISH)
            return fail(DC_ERR_UNSUPPORTED, "dc_add_group: item %d: activation id %d", i, it.activation);
        DC_REQUIRE_PTR("dc_add_group", it.a);
        DC_REQUIRE_PTR("dc_add_group", it.b);
        DC_REQUIRE_PTR("dc_add_group", it.out);
        DC_REQUIRE_PTR("dc_add_group", it.mask_a);
        DC_REQUIRE_PTR("dc_add_group", it.mask_b);
        DC_REQUIRE_PTR("dc_add_group", it.mask_out);
        if (it.activation > 0) DC_REQUIRE_PTR("dc_add_group", it.prev_out);
        DC_REQUIRE_ALIGNED("dc_add_group", it.a, esize(dtype));
        DC_REQUIRE_ALIGNED("dc_add_group", it.b, esize(dtype));
        DC_REQUIRE_ALIGNED("dc_add_group", it.out, esize(dtype));
        DC_REQUIRE_ALIGNED("dc_add_group", it.prev_out, esize(dtype));
        sums[i] = dc::AddGroupItem{it.a, it.b, it.activation > 0 ? it.prev_out : nullptr, it.out, it.mask_a, it.mask_b,
                                   it.mask_out, it.weight_a, it.weight_b, it.activation, it.batch, it.height, it.width,
                                   it.channels, it.scale};
    }
    for (int i = 0; i < count; ++i)
        for (int j = 0; j < count; ++j) {
            if (i == j) continue;
            const dc_add_item &a = items[i], &b = items[j];
            if (a.out == b.out || a.out == b.a || a.out == b.b || a.mask_out == b.mask_out || a.mask_out == b.mask_a ||
                a.mask_out == b.mask_b || (a.activation > 0 && b.activation > 0 && a.prev_out == b.prev_out))
                return fail(DC_ERR_UNSUPPORTED, "dc_add_group: items %d and %d share a buffer one of them writes", i, j);
        }
    if (!dc::add_group_eligible(sums, count, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_add_group: 16-bit types, channels %% 8 == 0, 16-byte aligned operands and "
                                        "maps below 2^18 pixels only");
    return finish(dc::launch_add_group(sums, count, dtype, (hipStream_t)stream), "dc_add_group");
}

int dc_pool_densify(const dc_geometry *g, const void *input, const int32_t *mask, void *prev_out,
                    void *out, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_pool_densify");
    int rc = check_geometry("dc_pool_densify", g, false, true);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_pool_densify", input);
    DC_REQUIRE_PTR("dc_pool_densify", mask);
    DC_REQUIRE_PTR("dc_pool_densify", prev_out);
    DC_REQUIRE_PTR("dc_pool_densify", out);
    DC_REQUIRE_ALIGNED("dc_pool_densify", prev_out, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_pool_densify", out, esize(dtype));
    if (!dc::pool_global_casts(*g, input, nullptr, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_pool_densify: needs a window covering the whole unpadded map, "
                                        "channels in whole 16-byte vectors and a 16-byte aligned input");
    return finish(dc::launch_pool_densify(*g, input, mask, prev_out, out, dtype, (hipStream_t)stream),
                  "dc_pool_densify");
}

int dc_linear(const void *x, const void *weight, const void *bias, void *out, int32_t rows,
              int32_t in_features, int32_t out_features, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_linear");
    if (rows <= 0 || in_features <= 0 || out_features <= 0)
        return fail(DC_ERR_SHAPE, "dc_linear: rows=%d in_features=%d out_features=%d must be positive", rows,
                    in_features, out_features);
    if ((int64_t)rows * in_features >= (int64_t)1 << 31 || (int64_t)rows * out_features >= (int64_t)1 << 31 ||
        (int64_t)in_features * out_features >= (int64_t)1 << 40)
        return fail(DC_ERR_SHAPE, "dc_linear: operands too large");
    if (!dc::linear_eligible(in_features, dtype))
        return fail(DC_ERR_UNSUPPORTED, "dc_linear: in_features=%d does not fill whole 16-byte vectors", in_features);
    DC_REQUIRE_PTR("dc_linear", x);
    DC_REQUIRE_PTR("dc_linear", weight);
    DC_REQUIRE_PTR("dc_linear", out);
    DC_REQUIRE_ALIGNED("dc_linear", x, 16);
    DC_REQUIRE_ALIGNED("dc_linear", weight, 16);
    DC_REQUIRE_ALIGNED("dc_linear", bias, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_linear", out, esize(dtype));
    return finish(dc::launch_linear(x, weight, bias, out, rows, in_features, out_features, dtype,
                                    (hipStream_t)stream), "dc_linear");
}

int dc_block(const dc_geometry *g, const dc_block_args *block, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_block");
    int rc = check_geometry("dc_block", g, false, false);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_block", block);
    const dc_block_args &b = *block;
    const char *why = dc::block_unsupported(*g, b, dtype);
    if (why != nullptr) return fail(DC_ERR_UNSUPPORTED, "dc_block: %s", why);
    DC_REQUIRE_PTR("dc_block", b.input);
    DC_REQUIRE_PTR("dc_block", b.mask);
    DC_REQUIRE_PTR("dc_block", b.dw_filter);
    DC_REQUIRE_PTR("dc_block", b.dw_prev_out);
    DC_REQUIRE_PTR("dc_block", b.dw_truncated);
    DC_REQUIRE_PTR("dc_block", b.project_packed_filter);
    DC_REQUIRE_PTR("dc_block", b.out);
    DC_REQUIRE_PTR("dc_block", b.out_mask);
    if (b.residual != nullptr) DC_REQUIRE_PTR("dc_block", b.residual_mask);
    if (b.expand_channels > 0) {
        DC_REQUIRE_PTR("dc_block", b.expand_packed_filter);
        DC_REQUIRE_PTR("dc_block", b.expand_prev_out);
        DC_REQUIRE_PTR("dc_block", b.expand_truncated);
        DC_REQUIRE_PTR("dc_block", b.expand_out);
        DC_REQUIRE_PTR("dc_block", b.expand_out_mask);
    }
    // 16-byte vectors on the depthwise side, 8-byte cells behind the matrix cores
    DC_REQUIRE_ALIGNED("dc_block", b.input, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.dw_filter, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.dw_prev_out, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.dw_truncated, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.project_packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.expand_packed_filter, 16);
    DC_REQUIRE_ALIGNED("dc_block", b.residual, 8);
    DC_REQUIRE_ALIGNED("dc_block", b.out, 8);
    DC_REQUIRE_ALIGNED("dc_block", b.expand_prev_out, 8);
    DC_REQUIRE_ALIGNED("dc_block", b.expand_truncated, 8);
    DC_REQUIRE_ALIGNED("dc_block", b.expand_out, 8);
    DC_REQUIRE_ALIGNED("dc_block", b.mask, 4);
    DC_REQUIRE_ALIGNED("dc_block", b.out_mask, 4);
    DC_REQUIRE_ALIGNED("dc_block", b.residual_mask, 4);
    DC_REQUIRE_ALIGNED("dc_block", b.expand_out_mask, 4);
    hipError_t e = dc::launch_block(*g, b, (hipStream_t)stream, &why);
    if (e == hipSuccess && why != nullptr) return fail(DC_ERR_UNSUPPORTED, "dc_block: %s", why);
    return finish(e, "dc_block");
}

int dc_add_to_dense(void *a, void *b, const int32_t *mask_a, int activation, int32_t pixels,
                    int32_t channels, int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_add_to_dense");
    int rc = check_pc("dc_add_to_dense", pixels, channels);
    if (rc != DC_OK) return rc;
    if (activation > DC_ACT_SWISH)
        return fail(DC_ERR_UNSUPPORTED, "dc_add_to_dense: activation id %d", activation);
    DC_REQUIRE_PTR("dc_add_to_dense", a);
    DC_REQUIRE_PTR("dc_add_to_dense", b);
    DC_REQUIRE_PTR("dc_add_to_dense", mask_a);
    DC_REQUIRE_ALIGNED("dc_add_to_dense", a, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_add_to_dense", b, esize(dtype));
    return finish(dc::launch_add_to_dense(a, b, mask_a, activation, pixels, channels, dtype,
                                          (hipStream_t)stream), "dc_add_to_dense");
}

int dc_upsample(const void *input, void *out, const int32_t *mask_in, int32_t *mask_out,
                int32_t batch, int32_t in_h, int32_t in_w, int32_t channels, int32_t scale,
                int dtype, void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_upsample");
    if (batch <= 0 || in_h <= 0 || in_w <= 0 || channels <= 0 || scale <= 0)
        return fail(DC_ERR_SHAPE, "dc_upsample: non-positive dimension");
    if ((int64_t)batch * in_h * in_w * scale * scale > (1 << 29))
        return fail(DC_ERR_SHAPE, "dc_upsample: more than 2^29 output pixels");
    DC_REQUIRE_PTR("dc_upsample", input);
    DC_REQUIRE_PTR("dc_upsample", out);
    DC_REQUIRE_PTR("dc_upsample", mask_in);
    DC_REQUIRE_PTR("dc_upsample", mask_out);
    DC_REQUIRE_ALIGNED("dc_upsample", input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_upsample", out, esize(dtype));
    return finish(dc::launch_upsample(input, out, mask_in, mask_out, batch, in_h, in_w, channels,
                                      scale, dtype, (hipStream_t)stream), "dc_upsample");
}

int dc_concat(const void *a, const void *b, void *out, const int32_t *mask_a, const int32_t *mask_b,
              int32_t *mask_out, int32_t pixels, int32_t channels_a, int32_t channels_b, int dtype,
              void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_concat");
    int rc = check_pc("dc_concat", pixels, channels_a);
    if (rc != DC_OK) return rc;
    rc = check_pc("dc_concat", pixels, channels_b);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_concat", a);
    DC_REQUIRE_PTR("dc_concat", b);
    DC_REQUIRE_PTR("dc_concat", out);
    DC_REQUIRE_PTR("dc_concat", mask_a);
    DC_REQUIRE_PTR("dc_concat", mask_b);
    DC_REQUIRE_PTR("dc_concat", mask_out);
    DC_REQUIRE_ALIGNED("dc_concat", a, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_concat", b, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_concat", out, esize(dtype));
    return finish(dc::launch_concat(a, b, out, mask_a, mask_b, mask_out, pixels, channels_a,
                                    channels_b, dtype, (hipStream_t)stream), "dc_concat");
}

int dc_mul_add(const void *input, const int32_t *mask, void *out, int32_t *mask_out,
               const void *scale, const void *bias, int32_t pixels, int32_t channels, int dtype,
               void *stream) {
    dc::kernel_log_reset();
    DC_REQUIRE_DTYPE("dc_mul_add");
    int rc = check_pc("dc_mul_add", pixels, channels);
    if (rc != DC_OK) return rc;
    DC_REQUIRE_PTR("dc_mul_add", input);
    DC_REQUIRE_PTR("dc_mul_add", mask);
    DC_REQUIRE_PTR("dc_mul_add", out);
    DC_REQUIRE_PTR("dc_mul_add", mask_out);
    DC_REQUIRE_PTR("dc_mul_add", scale);
    DC_REQUIRE_ALIGNED("dc_mul_add", input, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_mul_add", out, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_mul_add", scale, esize(dtype));
    DC_REQUIRE_ALIGNED("dc_mul_add", bias, esize(dtype));
    return finish(dc::launch_mul_add(input, mask, out, mask_out, scale, bias, pixels, channels,
                                     dtype, (hipStream_t)stream), "dc_mul_add");
}

}  // extern "C"
