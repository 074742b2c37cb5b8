/*
 * deltacnn_hip.h -- C ABI of libdeltacnn_hip.so: DeltaCNN's sparse delta-propagation
 * operators as hand-written gfx950 (MI355X) HIP kernels.
 *
 * Every entry point replaces one function of the reference's pybind11 module
 * `deltacnn.cuda` (src/cuda/conv_torch_wrapper.cpp:640-655).  Conventions:
 *
 *   - feature tensors are NHWC (torch.channels_last) device pointers, element type
 *     given by `dtype` (DC_F32, DC_F16 or DC_BF16); masks are dense int32 [B*H*W] device
 *     pointers, a pixel is active iff its word != 0
 *   - the library never allocates, frees or retains memory; pointers are borrowed
 *     for the duration of the asynchronous launch on `stream` (a hipStream_t, NULL =
 *     default stream); no entry point synchronises
 *   - values of inactive pixels never influence any output (they may hold anything,
 *     NaN included; a kernel may load them speculatively, always inside the tensor,
 *     and discards them); outputs are written only for pixels whose output mask is 1
 *     (the reference additionally writes the inactive pixels of partially active
 *     tiles, conv_kernel.cu:348-356; nothing downstream reads them)
 *   - return value: DC_OK or a negative dc_status; dc_last_error() gives the message
 *     of the calling thread's last failure.  All argument checks run before the first
 *     HIP call, so they can be exercised without a GPU.
 */
#ifndef DELTACNN_HIP_H
#define DELTACNN_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum dc_status {
    DC_OK = 0,
    DC_ERR_DTYPE = -1,       /* dtype not DC_F32 / DC_F16 / DC_BF16 */
    DC_ERR_SHAPE = -2,       /* non-positive or inconsistent dimensions */
    DC_ERR_UNSUPPORTED = -3, /* valid but not implemented configuration */
    DC_ERR_NULL = -4,        /* required pointer is NULL */
    DC_ERR_ALIGN = -5,       /* pointer not aligned to its element / vector size */
    DC_ERR_LAUNCH = -6       /* HIP reported a launch error */
} dc_status;

/* DC_BF16: bfloat16 has no counterpart in the reference (readme.md:228, fp16 and fp32 only); every
 * operator follows the fp16 rules with two exceptions: sparsify compares with > for any channel
 * count, and filters use the fp32 layout [Cin/g][Kh][Kw][Cout] (no padding, no pair swizzle). */
enum { DC_F32 = 0, DC_F16 = 1, DC_BF16 = 2 };

/* activation ids of convert_activation_string (sparse_layers.py:20-34); <= 0 is linear */
enum { DC_ACT_LINEAR = 0, DC_ACT_RELU = 1, DC_ACT_RELU6 = 2, DC_ACT_LEAKY = 3,
       DC_ACT_SIGMOID = 4, DC_ACT_SWISH = 5 };

/* DCTruncation (sparse_layers.py:102-106) */
enum { DC_TRUNC_NONE = -1, DC_TRUNC_MAX = 0, DC_TRUNC_NORM = 1, DC_TRUNC_RMS = 2 };

/* pooling_mode of sparse_pooling_wrapper_masked (conv_torch_wrapper.cpp:213-226) */
enum { DC_POOL_MAX = 0, DC_POOL_AVG = 1 };

/* Geometry of a (transposed) convolution or pooling window.  Mirrors the reference's
 * Dimensions + ConvConfig structs (src/cuda/common.cuh:12-35) with 32-bit fields and
 * padding in (top, left, bottom, right) order like conv_torch_wrapper.cpp:43-53. */
typedef struct dc_geometry {
    int32_t batch;
    int32_t in_h, in_w, in_c;
    int32_t out_h, out_w, out_c;
    int32_t kernel_h, kernel_w;
    int32_t stride_h, stride_w;
    int32_t dilation_h, dilation_w;
    int32_t pad_top, pad_left, pad_bottom, pad_right;
    int32_t groups;
} dc_geometry;

const char *dc_version(void);
const char *dc_last_error(void);

/* Names of the kernels that the calling thread's last entry point launched, '+'-separated
 * (e.g. "pw_mfma_kernel+act_trunc_vec_kernel"); empty if it launched nothing.  For tracing
 * tools; no counterpart in the reference. */
const char *dc_last_kernels(void);

/* Replaces deltacnn_prepare_diff_mask_wrapper (conv_torch_wrapper.cpp:347-384).
 * delta = input - prev_input; active pixels get delta and prev_input := input on all
 * channels; mask is written for every pixel. */
int dc_sparsify(const void *input, void *prev_input, void *delta, int32_t *mask,
                float threshold, int32_t pixels, int32_t channels, int dtype, void *stream);

/* Replaces deltacnn_activate_truncate (conv_torch_wrapper.cpp:295-344).  In place on delta,
 * prev_input, truncated and mask.  truncation_mode < 0 accumulates delta into prev_input
 * (densify); `truncated` may then be NULL. */
int dc_activate_truncate(void *delta, void *prev_input, void *truncated, int32_t *mask,
                         float threshold, int activation, int truncation_mode,
                         int32_t pixels, int32_t channels, int dtype, void *stream);

/* Replaces sparse_conv_bias_wrapper_masked (conv_torch_wrapper.cpp:62-134).
 * `filter` is in the reference layout produced by process_filters(): fp32
 * [Cin/g][Kh][Kw][Cout]; fp16 the same with Cin and Cout padded to even and the 2x2
 * channel-pair swizzle of filter_conversion.py:13-38 (depthwise: unpadded, unswizzled).
 * `packed_filter` (optional, may be NULL) is the output of dc_pack_filter for the same
 * filter; when given, eligible shapes run on the MFMA kernels.
 * `bias` may be NULL.  groups must be 1 or in_c == out_c (depthwise). */
int dc_conv(const dc_geometry *g, const void *input, const void *filter,
            const void *packed_filter, const void *bias, void *out, const int32_t *mask,
            int32_t *out_mask, int dtype, void *stream);

/* Conv + activation/truncation in one call: dc_conv followed by dc_activate_truncate on the
 * conv output.  Depthwise, few-input-channel, mid-size pointwise and small KxK shapes of up
 * to 32 output channels, K x K layers with 8 / 16 input channels on large maps, and larger K x K
 * layers of up to 64 output channels on at most 256 output tiles of 8 x 8 run as ONE launch
 * (the epilogue works on the accumulators, the conv output never travels through memory; `out`
 * then holds the activated difference of the pixels whose out_mask word is set and is undefined
 * elsewhere, as after the two calls);
 * every other shape runs the two kernels back to back inside the call.  No counterpart in
 * the reference (it launches the two kernels separately, sparse_layers.py:636-638); results
 * are identical to the two-call sequence bit for bit. */
int dc_conv_act(const dc_geometry *g, const void *input, const void *filter,
                const void *packed_filter, const void *bias, void *out, const int32_t *mask,
                int32_t *out_mask, void *prev_out, void *truncated, float threshold,
                int activation, int truncation_mode, int dtype, void *stream);

/* Fused conv + residual add: the DCAdd (sparse_layers.py:1086-1182, not dense_out) that follows a
 * block's last convolution, in the convolution's launch: with a = residual, b = conv(input),
 * s = weight_residual * a [mask_residual] + weight_conv * b [mask]; activation == 0: out = s;
 * activation > 0 (other_nn_layers.cu:1379-1559): prev_out += s, out = act(prev_out) - act(old
 * prev_out).  out_mask = mask | mask_residual.  Results are identical to dc_conv followed by
 * dc_add(residual, conv).  No counterpart in the reference.  For the 16-bit types: 1x1 stride-1
 * convolutions without padding (Cin % 8 == 0, Cout % 4 == 0), and K x K layers (Cin % 8 == 0,
 * groups 1, at most 64 taps) whose input window of an 8 x 8 output tile fits the kernel's LDS
 * staging (any layer of up to 32 x 32 halo pixels does), with or
 * without activation (layers beyond ceil(W/4) * ceil(H/4) * B * ceil(Cout/16) * Kh * Kw *
 * ceil(Cin/32) = 32768: without activation only).  All need a packed filter; anything else returns DC_ERR_UNSUPPORTED before any
 * launch so that the caller can issue the two separate calls.  prev_out may be NULL when
 * activation == 0. */
int dc_conv_add(const dc_geometry *g, const void *input, const void *packed_filter,
                const void *bias, const int32_t *mask, const void *residual,
                const int32_t *mask_residual, void *out, int32_t *out_mask, float weight_residual,
                float weight_conv, void *prev_out, int activation, int dtype, void *stream);

/* Operands of dc_block beyond the depthwise geometry.  Feature pointers are fp16 NHWC; the
 * packed filters come from dc_pack_filter (1x1 geometry of that convolution). */
typedef struct dc_block_args {
    /* A: depthwise 3x3 convolution (geometry argument) + activation/truncation */
    const void *input;              /* [B][in_h][in_w][C] delta */
    const int32_t *mask;            /* its update mask */
    const void *dw_filter;          /* reference depthwise layout [3][3][C] */
    void *dw_prev_out;              /* activation state [B][out_h][out_w][C], in place */
    void *dw_truncated;
    float dw_threshold;
    int32_t dw_activation;          /* DC_ACT_RELU / RELU6 / LEAKY */
    int32_t dw_truncation_mode;     /* DC_TRUNC_MAX */
    /* B: 1x1 projection C -> project_channels (+ residual sum, a DCAdd without activation) */
    const void *project_packed_filter;
    int32_t project_channels;
    const void *residual;           /* [P][project_channels] delta or NULL */
    const int32_t *residual_mask;   /* required with residual */
    float weight_residual, weight_conv;
    void *out;                      /* [P][project_channels], written where out_mask is 1 */
    int32_t *out_mask;              /* [P], written for every pixel */
    /* C (expand_channels > 0): 1x1 expansion project_channels -> expand_channels + activation/truncation */
    const void *expand_packed_filter;
    int32_t expand_channels;
    void *expand_prev_out;          /* [P][expand_channels], in place */
    void *expand_truncated;
    float expand_threshold;
    int32_t expand_activation;      /* must equal dw_activation */
    int32_t expand_truncation_mode; /* DC_TRUNC_MAX */
    void *expand_out;               /* [P][expand_channels], written where expand_out_mask is 1 */
    int32_t *expand_out_mask;       /* [P], written for every pixel */
    int32_t flags;                  /* DC_BLOCK_* bits */
} dc_block_args;

/* dc_block_args.flags.  By default layers with small filters request every operand before the
 * update masks are known (one memory round trip; what was fetched for inactive pixels is
 * dropped): right for small batches, which are bound by latency.  DC_BLOCK_LATE_LOADS fetches
 * only what active pixels need, one round trip later: right when the maps are large and mostly
 * inactive.  Results do not depend on it. */
enum { DC_BLOCK_LATE_LOADS = 1 };

/* The layers between two spatial convolutions of an inverted-residual network in ONE launch:
 * depthwise 3x3 convolution + activation/truncation, 1x1 projection (+ residual sum) and,
 * optionally, the next block's 1x1 expansion + activation/truncation.  `g` describes the
 * depthwise convolution (groups == in_c == out_c); P = batch * out_h * out_w.  Neither the
 * depthwise output nor, on its way into the expansion, the block output passes through memory.
 * Results (all outputs, masks and layer states) are identical, bit for bit, to
 * dc_conv_act(depthwise) -> dc_conv / dc_conv_add(projection) -> dc_conv_act(expansion), none
 * of them with a bias (a layer's bias belongs to its first frame, which takes the separate
 * calls).  fp16 only.  Shapes outside the kernel's range (see dc_last_error) return
 * DC_ERR_UNSUPPORTED before any launch so that the caller can issue the separate calls.  No
 * counterpart in the reference, which launches every layer and every activation on its own
 * (sparse_layers.py:636-638). */
int dc_block(const dc_geometry *g, const dc_block_args *block, int dtype, void *stream);

/* Operands of dc_expand_depthwise beyond the depthwise geometry. */
typedef struct dc_expand_dw_args {
    /* A: 1x1 expansion expand_in_channels -> C (the depthwise layer's channels) + activation/truncation */
    const void *input;              /* [B][H][W][expand_in_channels] delta */
    const int32_t *mask;            /* its update mask */
    const void *expand_packed_filter; /* NULL: dc_project_expand already ran the convolution (input, mask unused) */
    int32_t expand_in_channels;
    void *expand_prev_out;          /* [P][C] activation state of the expansion, in place */
    void *expand_truncated;
    float expand_threshold;
    int32_t expand_activation;
    int32_t expand_truncation_mode; /* DC_TRUNC_MAX */
    void *expand_out;               /* [P][C] the expansion's output delta, valid on the pixels it keeps */
    int32_t *expand_out_mask;       /* [P] receives the UPDATE mask of the expansion's convolution (= mask) */
    /* B: depthwise 3x3, stride 1 or 2, padding 1 (geometry argument) + activation/truncation */
    const void *dw_filter;          /* reference depthwise layout [3][3][C] */
    void *dw_prev_out;              /* [P][C], in place */
    void *dw_truncated;
    float dw_threshold;
    int32_t dw_activation;
    int32_t dw_truncation_mode;
    void *out;                      /* [P][C], written where out_mask is 1 */
    int32_t *out_mask;              /* [P], written for every pixel */
} dc_expand_dw_args;

/* A 1x1 expansion with activation / maximum-norm truncation followed by a depthwise 3x3
 * (stride 1 or 2, padding 1) with activation / truncation, as two launches instead of three: the
 * expansion's convolution computes T = truncated + v, S = T + prev, D = act(S) - act(prev) for
 * every updated pixel, stores D and T, and leaves the keep decision -- any |D| of a pixel's
 * channels above the threshold, which no workgroup of that kernel can see -- to the depthwise
 * kernel, whose lane groups read whole pixel rows anyway: a window pixel counts only if the
 * decision holds for it, and every group commits the expansion's state of the input pixels it
 * owns (stride 1: its centre pixel; stride 2: the 2 x 2 block at twice its output coordinates).
 * All layer states and the depthwise output are identical, bit for bit, to
 * dc_conv_act(expansion) followed by dc_conv_act(depthwise); of the expansion's own output only
 * the pixels it keeps are meaningful (as always), and expand_out_mask receives its convolution's
 * update mask rather than the keep mask.  For the small maps where launches are the cost:
 * shapes outside the range (see dc_last_error) return DC_ERR_UNSUPPORTED before any launch so
 * that the caller can issue the separate calls.  16-bit types, the expansion's output channels in
 * multiples of 8; no bias (a layer's bias belongs
 * to its first frame, which takes the separate calls).  No counterpart in the reference, which
 * launches every layer and every activation on its own (sparse_layers.py:636-638). */
int dc_expand_depthwise(const dc_geometry *g, const dc_expand_dw_args *args, int dtype, void *stream);

/* Operands of dc_project_expand beyond the projection's 1x1 geometry. */
typedef struct dc_project_expand_args {
    /* A: 1x1 projection in_c -> out_c of the geometry argument, no activation */
    const void *input;              /* [P][in_c] delta (the block's depthwise output) */
    const int32_t *mask;            /* its update mask */
    const void *project_packed_filter;
    const void *residual;           /* [P][out_c] delta added to the projection (DCAdd without activation), or NULL */
    const int32_t *residual_mask;
    float weight_residual, weight_conv;
    void *out;                      /* [P][out_c] block output delta, written where out_mask is 1 */
    int32_t *out_mask;              /* [P] = mask | residual_mask, written for every pixel */
    /* B: 1x1 expansion out_c -> expand_channels of the next block, activation left open */
    const void *expand_packed_filter;
    int32_t expand_channels;
    void *expand_prev_out;          /* [P][expand_channels] accumulated values: read only in this call */
    void *expand_truncated;         /* receives T = truncated + v on updated pixels */
    int32_t expand_activation;      /* DC_ACT_RELU or DC_ACT_RELU6 */
    void *expand_out;               /* [P][expand_channels] receives D = act(T + prev) - act(prev) on updated pixels */
    int32_t *expand_out_mask;       /* [P] receives the update mask (= out_mask) */
    /* C: the depthwise layer that will finish the expansion (checked, not run) */
    const dc_geometry *dw_geometry;
    int32_t dw_activation;
    int32_t dw_truncation_mode;
} dc_project_expand_args;

/* The 1x1 projection that ends an inverted-residual block (with the block's residual sum) and the
 * 1x1 expansion that starts the next block in ONE launch, for the small maps where launches are
 * the cost.  The expansion's activation is left open exactly as the first launch of
 * dc_expand_depthwise leaves it (D and T stored, accumulated values untouched); the NEXT call on
 * these buffers has to be dc_expand_depthwise with expand_packed_filter == NULL, which runs only
 * its second launch -- the depthwise kernel that takes the keep decision and commits the
 * expansion's state.  This call verifies that that call will be accepted (dw_geometry,
 * dw_activation, dw_truncation_mode) and returns DC_ERR_UNSUPPORTED before any launch otherwise,
 * as for shapes outside its own range: block output channels in multiples of 32 up to 96, a
 * projection filter of at most 128 KB (every workgroup streams it), layers small enough that the
 * stand-alone pointwise kernel would split the projection's reduction over four wavefronts and
 * the expansion's over none.  Together the two calls are identical, bit for bit, to
 * dc_conv / dc_conv_add(projection), dc_conv_act(expansion), dc_conv_act(depthwise).  16-bit
 * types; no bias.  Several workgroups per pixel tile read every input of the call while one of
 * them stores the block output, so nothing is summed in place: out, out_mask, expand_out,
 * expand_out_mask and expand_truncated must not overlap input, mask, residual, residual_mask,
 * expand_prev_out, the filters or one another (DC_ERR_UNSUPPORTED otherwise).  No counterpart in
 * the reference (sparse_layers.py:636-638). */
int dc_project_expand(const dc_geometry *g, const dc_project_expand_args *args, int dtype, void *stream);

/* One layer of a dc_conv_group call. */
typedef struct dc_conv_item {
    dc_geometry geometry;           /* 3x3 or 1x1 convolution, groups == 1 */
    const void *input;              /* [B][in_h][in_w][in_c] delta */
    const int32_t *mask;            /* its update mask */
    const void *packed_filter;      /* from dc_pack_filter */
    const void *bias;               /* [out_c] or NULL */
    void *out;                      /* [B][out_h][out_w][out_c] */
    int32_t *out_mask;              /* [B][out_h][out_w] */
    /* the residual sum of dc_conv_add behind the convolution; residual == NULL: none */
    const void *residual;
    const int32_t *residual_mask;
    float weight_residual, weight_conv;
    void *sum_prev_out;             /* accumulated sum of a DCAdd with activation (sum_activation > 0) */
    int32_t sum_activation;
    /* the activation / truncation of dc_conv_act behind the convolution; prev_out == NULL: none.
     * Not together with a residual sum. */
    void *prev_out;
    void *truncated;
    float threshold;
    int32_t activation;
    int32_t truncation_mode;        /* DC_TRUNC_MAX */
} dc_conv_item;

enum { DC_CONV_GROUP_MAX = 8 };

/* 2 .. DC_CONV_GROUP_MAX independent small layers -- the parallel branches of a
 * multi-resolution network, whose layers the reference (and dc_conv / dc_conv_act / dc_conv_add)
 * launch one after the other -- in ONE launch, plus one more for the activation / truncation of
 * those items whose convolution cannot finish it itself.  Each item is what one call of dc_conv,
 * dc_conv_act or dc_conv_add would be given, and its results are identical, bit for bit, to that
 * call's.  The items must not depend on each other (no item's output or state is another's
 * operand).  Accepted, for the 16-bit types: either 3x3 kernels on layers small enough for the
 * library's 4x4-patch kernel, with activations of maximum-norm truncation, all of one kind where
 * they need the second launch; or plain 1x1 stride-1 convolutions (no residual sum, no
 * activation) on maps below 2^16 pixels with a reduction of at most 10 steps of 32 channels (or
 * 1024 output tiles of 16 x 16 and more), the layers the library runs one wavefront per tile.
 * Anything else, and a mix of the two, returns DC_ERR_UNSUPPORTED before any launch so that the
 * caller can issue the separate calls.  No counterpart in the reference
 * (sparse_layers.py:425-470 runs one layer per call). */
int dc_conv_group(const dc_conv_item *items, int32_t count, int dtype, void *stream);

/* One sum of a dc_add_group call: the arguments of dc_add_upsampled (scale 1: those of dc_add
 * without dense_out). */
typedef struct dc_add_item {
    const void *a;                  /* [B][H][W][C] delta */
    const void *b;                  /* [B][H/scale][W/scale][C] delta */
    void *prev_out;                 /* accumulated sum (activation > 0), or NULL */
    void *out;                      /* [B][H][W][C] */
    const int32_t *mask_a, *mask_b;
    int32_t *mask_out;              /* [B][H][W] = mask_a | upsampled mask_b */
    float weight_a, weight_b;
    int32_t activation;
    int32_t batch, height, width, channels, scale;
} dc_add_item;

/* 2 .. DC_CONV_GROUP_MAX independent sums -- those of one level of a multi-resolution exchange,
 * which the reference launches one after the other (sparse_layers.py:1086-1182) -- in ONE launch.
 * Each item's results are identical, bit for bit, to dc_add_upsampled's (dc_add's for scale 1).
 * No item's output, mask or accumulated sum may be another's operand.  For the 16-bit types,
 * channels in multiples of 8, 16-byte aligned operands and maps below 2^18 pixels; anything else
 * returns DC_ERR_UNSUPPORTED before any launch so that the caller can issue the separate calls.
 * No counterpart in the reference. */
int dc_add_group(const dc_add_item *items, int32_t count, int dtype, void *stream);

/* Number of bytes dc_pack_filter writes for this geometry (0 if the shape has no packed
 * form).  One-time weight relayout for the MFMA kernels, fp16 or bfloat16, un-swizzled, in fragment order
 * [Cout tile of 16][Kh][Kw][Cin step of 32][lane 0..63][8] (lane kq*16+r holds input channels
 * kq*8..+8 of output channel r): round_up(Cout,16) * Kh * Kw * round_up(Cin,32) halves.
 * Stems (Cin <= 4, window up to 8 x 8, Cout <= 64 and a multiple of 4, not transposed) pack as
 * [Cout tile of 16][Kh][lane][8] with reduction element k = kx * 4 + ci of a window row,
 * ceil(Cout / 16) * Kh * 512 halves.  The buffer is opaque to callers: only dc_pack_filter
 * writes it and only this library reads it; it has to be made from the same Cin, Cout and
 * window as the convolution it is handed to. */
int64_t dc_packed_filter_bytes(const dc_geometry *g, int dtype, int transposed);
int dc_pack_filter(const dc_geometry *g, const void *filter, void *packed_filter, int dtype,
                   int transposed, void *stream);

/* Replaces sparse_deconv_bias_wrapper_masked (conv_torch_wrapper.cpp:136-210).  `filter`
 * layout [Cin][Kh][Kw][Cout] (fp16: padded + swizzled as for dc_conv).  Any kernel size /
 * stride with groups == 1 (the reference supports only k4s2 and k6s4,
 * deconv_kernel.cu:857,872). */
int dc_deconv(const dc_geometry *g, const void *input, const void *filter,
              const void *packed_filter, const void *bias, void *out, const int32_t *mask,
              int32_t *out_mask, int dtype, void *stream);

/* dc_deconv followed by dc_add(deconv, residual) -- the DCAdd (sparse_layers.py:1086-1182, no
 * activation, no dense_out) that merges an up-sampled level into the next one -- in the transposed
 * convolution's launch: out = weight_residual * residual [mask_residual] + weight_conv *
 * deconv(input) [updated pixels], out_mask = the union, with the arithmetic of dc_conv_add
 * (activation 0), whose results it equals bit for bit.  16-bit types, groups 1, dilation 1,
 * Cin % 8 == 0, a window at least as large as the stride, layers beyond the 4 x 4-patch kernel's
 * range (the other transposed layers return DC_ERR_UNSUPPORTED before any launch, and the caller
 * issues the two calls); no bias (it belongs to the first frame).  out and out_mask must not
 * overlap the operands.  No counterpart in the reference, which launches deconv_kernel.cu's
 * kernel and the addition separately (sparse_layers.py:1101-1174). */
int dc_deconv_add(const dc_geometry *g, const void *input, const void *packed_filter, const int32_t *mask,
                  const void *residual, const int32_t *mask_residual, void *out, int32_t *out_mask,
                  float weight_residual, float weight_conv, int dtype, void *stream);

/* Replaces sparse_pooling_wrapper_masked (conv_torch_wrapper.cpp:213-293).  `prev_input` is
 * required for DC_POOL_MAX.  When out_h == out_w == 1, `out` is [B][C], fully overwritten, of
 * type `global_out_dtype`: DC_F32 is the reference's protocol (a float32 accumulator,
 * cuda_kernels.py:101-109, cast back by the caller, :123-124); passing `dtype` fuses that
 * cast (window == whole unpadded map, channels a multiple of the 16-byte vector, else
 * DC_ERR_UNSUPPORTED before any launch).  Ignored for other output sizes. */
int dc_pool(const dc_geometry *g, const void *input, const void *prev_input, void *out,
            const int32_t *mask, int32_t *out_mask, int pooling_mode, int dtype,
            int global_out_dtype, void *stream);

/* A 1x1 convolution (stride 1, no padding, no bias) over the concatenation, along the channels,
 * of `count` (2..4) delta tensors that is never formed: DCConcatenate (sparse_layers.py:1185-1194,
 * other_nn_layers.cu:3601-3771) chained count - 1 times, then dc_conv, in the convolution's
 * launch.  `g` describes the convolution of the concatenated tensor (in_c = the sum of
 * `channels`); inputs[i] is [B][H][W][channels[i]] with update mask masks[i].  A pixel takes part
 * in the reduction steps of tensor i only where masks[i] is set -- where the concatenation would
 * hold zeros -- and out_mask is the union of the masks, so out and out_mask equal those of the
 * separate calls bit for bit (the launch uses the arrangement, and hence the summation order,
 * dc_conv picks for the concatenated layer).  16-bit types, channels[i] in multiples of 32,
 * out_c % 4 == 0, a packed filter of the whole layer; anything else returns DC_ERR_UNSUPPORTED
 * before any launch so that the caller can issue the separate calls.  No counterpart in the
 * reference, which launches every concatenation (sparse_layers.py:1185-1194). */
int dc_concat_conv(const dc_geometry *g, int32_t count, const void *const *inputs, const int32_t *const *masks,
                   const int32_t *channels, const void *packed_filter, void *out, int32_t *out_mask, int dtype,
                   void *stream);

/* Maximum pooling of a DCMaxPooling layer together with the update of its cached input
 * (sparse_layers.py:1466-1468: the pooling call, then prev_in[mask] += delta) in ONE launch:
 * dc_pool(DC_POOL_MAX) followed by dc_add_to_dense(input, prev_input, mask), with identical
 * results.  For windows that tile the map exactly -- 2x2 or 3x3, stride == window, no padding,
 * no dilation, input size = output size * stride -- so that every input pixel belongs to one
 * window and its owner can update it; channels in whole 16-byte vectors, 16-byte aligned
 * tensors, at most 2^20 lanes (output pixels x lanes per pixel).  Other shapes return
 * DC_ERR_UNSUPPORTED before any launch and the caller issues the two calls.  prev_input is
 * updated in place; out and out_mask must not overlap it or the inputs. */
int dc_pool_update(const dc_geometry *g, const void *input, void *prev_input, void *out, const int32_t *mask,
                   int32_t *out_mask, int dtype, void *stream);

/* Replaces sparse_add_tensors_wrapper (conv_torch_wrapper.cpp:387-444). */
int dc_add(const void *a, const void *b, void *prev_out, void *out, const int32_t *mask_a,
           const int32_t *mask_b, int32_t *mask_out, float weight_a, float weight_b,
           int activation, int dense_out, int32_t pixels, int32_t channels, int dtype,
           void *stream);

/* dc_add whose operand b lives on a map `scale` times smaller in both directions and enters
 * through nearest upsampling: out(y, x) = weight_a * a(y, x) + weight_b * b(y / scale, x / scale),
 * mask_out = mask_a | upsampled mask_b.  height and width are those of a and out and must be
 * multiples of scale; no dense_out form.  No counterpart in the reference, which runs
 * sparse_upsample_wrapper (conv_torch_wrapper.cpp:484-513) and sparse_add_tensors_wrapper
 * (:387-444) one after the other; results are identical, the upsampled tensor is never stored. */
int dc_add_upsampled(const void *a, const void *b, void *prev_out, void *out, const int32_t *mask_a,
                     const int32_t *mask_b, int32_t *mask_out, float weight_a, float weight_b,
                     int activation, int32_t batch, int32_t height, int32_t width, int32_t channels,
                     int32_t scale, int dtype, void *stream);

/* DCDensify in one launch (sparse_layers.py:1287-1329): prev_out += delta on active pixels,
 * then out = prev_out for EVERY pixel (the dense clone of :1324-1325).  No counterpart in the
 * reference, which runs deltacnn_activate_truncate(..., truncation_mode -1) and a torch clone;
 * results are identical. */
int dc_densify(const void *delta, void *prev_out, void *out, const int32_t *mask, int32_t pixels,
               int32_t channels, int dtype, void *stream);

/* The tail of a classification network in one launch: global average pooling over the whole
 * unpadded map (sparse_pooling_wrapper_masked with a 1x1 output, conv_torch_wrapper.cpp:213-293)
 * followed by DCDensify (sparse_layers.py:1287-1329) on its one-pixel result: with
 * d = mean of the deltas of the map's updated pixels, rounded to the tensor type, prev_out += d
 * if any pixel was updated, out = prev_out.  input is [B, H, W, C] with g->in_h x g->in_w the
 * window, prev_out and out are [B, C].  Results are identical to dc_pool (mode average, output
 * in the tensor type) followed by dc_densify; the pooled delta and its mask are not stored.
 * Needs C in whole 16-byte vectors and a 16-byte aligned input, else DC_ERR_UNSUPPORTED before
 * any launch (the caller then issues the two calls).  No counterpart in the reference. */
int dc_pool_densify(const dc_geometry *g, const void *input, const int32_t *mask, void *prev_out,
                    void *out, int dtype, void *stream);

/* Dense layer on a few rows: out[r][o] = bias[o] + sum_i x[r][i] * weight[o][i], weight in
 * torch.nn.Linear's [out_features][in_features] layout, bias may be NULL; fp32 accumulation
 * in a fixed order, one rounding.  For the classifier behind DCDensify, which the reference
 * leaves to torch (example/mobilenet_deltacnn.py:196-199, 225): at one row per stream it is a
 * matrix-vector product of launch-latency size.  in_features must fill whole 16-byte vectors
 * (DC_ERR_UNSUPPORTED otherwise); x, weight 16-byte aligned.  No counterpart in the reference. */
int dc_linear(const void *x, const void *weight, const void *bias, void *out, int32_t rows,
              int32_t in_features, int32_t out_features, int dtype, void *stream);

/* Replaces sparse_add_to_dense_tensor_wrapper (conv_torch_wrapper.cpp:447-482):
 * b[px] += a[px] on active pixels.  With activation > 0 it also writes a = act(b) on every
 * pixel (the USE_ACTIVATION variant, other_nn_layers.cu:1731-1957). */
int dc_add_to_dense(void *a, void *b, const int32_t *mask_a, int activation, int32_t pixels,
                    int32_t channels, int dtype, void *stream);

/* Replaces sparse_upsample_wrapper (conv_torch_wrapper.cpp:484-522): nearest upsample by an
 * integer factor. */
int dc_upsample(const void *input, void *out, const int32_t *mask_in, int32_t *mask_out,
                int32_t batch, int32_t in_h, int32_t in_w, int32_t channels, int32_t scale,
                int dtype, void *stream);

/* Replaces sparse_concatenate_wrapper (conv_torch_wrapper.cpp:524-567). */
int dc_concat(const void *a, const void *b, void *out, const int32_t *mask_a,
              const int32_t *mask_b, int32_t *mask_out, int32_t pixels, int32_t channels_a,
              int32_t channels_b, int dtype, void *stream);

/* Replaces sparse_mul_add_wrapper (conv_torch_wrapper.cpp:569-630): out = in*scale (+bias)
 * per channel on active pixels; mask_out := mask when they are distinct buffers. */
int dc_mul_add(const void *input, const int32_t *mask, void *out, int32_t *mask_out,
               const void *scale, const void *bias, int32_t pixels, int32_t channels,
               int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DELTACNN_HIP_H */
