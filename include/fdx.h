/*
 * fdx -- C ABI of the MI355X (gfx950) forward path for frugally-deep models.
 *
 * Everything behind fdeep::load_model / model::predict / predict_multi runs through
 * these entry points: the C++ facade in include/fdeep/fdeep.hpp, the ctypes
 * binding and the tests call nothing else.  Plain pointers and sizes only.
 *
 * Conventions
 *   - every function returns fdx_status, 0 = ok; fdx_last_error() gives the text
 *     (thread-local), which the C++ facade rethrows as std::runtime_error the way
 *     include/fdeep/common.hpp:42-57 raises.
 *   - tensors are fp32, channels-last, batch outermost: [n][h][w][c] / [n][rows][depth].
 *   - "dev" pointers are device memory of the current GPU; the per-kernel launchers
 *     take device pointers only and enqueue on the library stream (fdx_sync waits).
 *   - host threads: every call enqueues on the one library stream, so work from several
 *     threads runs in the order the calls were made; a model (and a session) serialises
 *     its own calls, the convolution / GEMM launcher serialises its tuner and scratch.
 *   - measurement aids and test hooks (stopwatch, per-kernel profile, shader-clock probe, forced kernel choices) are
 *     declared apart, in fdx_debug.h: nothing a caller of the reference's API needs.
 */
#ifndef FDX_H
#define FDX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int fdx_status;
enum { FDX_OK = 0, FDX_ERR_INVALID = 1, FDX_ERR_HIP = 2, FDX_ERR_FORMAT = 3, FDX_ERR_UNSUPPORTED = 4 };

/* Activations.  NONE / RELU / GELU may be fused into any producer's epilogue; the others run through
 * fdx_activation_f32 (the launchers that take an epilogue activation reject them).  Formulas as in
 * include/fdeep/recurrent_ops.hpp:24-86 and include/fdeep/layers/<name>_layer.hpp; the three float fields
 * carry each kind's parameters:
 *   RELU         max_value, negative_slope, threshold            (relu_layer.hpp:40-46)
 *   ELU / CELU   negative_slope = alpha: x >= 0 ? x : alpha * (e^x - 1)
 *   LEAKY_RELU   negative_slope: x > 0 ? x : slope * x
 *   HARD_SHRINK  threshold: |x| > thr ? x : 0          SOFT_SHRINK  threshold: x -+ thr or 0
 *   SQUARE_PLUS  max_value = b: (x + sqrt(x^2 + b)) / 2
 *   THRESHOLD    threshold, max_value = default value: x > thr ? x : default
 *   LOG          natural logarithm (second half of log_softmax = log(softmax(x)), log_softmax_layer.hpp) */
enum {
    FDX_ACT_NONE = 0, FDX_ACT_RELU = 1, FDX_ACT_GELU = 2,
    FDX_ACT_TANH = 3, FDX_ACT_SIGMOID = 4, FDX_ACT_SWISH = 5, FDX_ACT_HARD_SIGMOID = 6, FDX_ACT_SELU = 7, FDX_ACT_ELU = 8,
    FDX_ACT_EXPONENTIAL = 9, FDX_ACT_SOFTSIGN = 10, FDX_ACT_SOFTPLUS = 11, FDX_ACT_LEAKY_RELU = 12, FDX_ACT_HARD_SHRINK = 13,
    FDX_ACT_SOFT_SHRINK = 14, FDX_ACT_SPARSE_PLUS = 15, FDX_ACT_SQUARE_PLUS = 16, FDX_ACT_TANH_SHRINK = 17,
    FDX_ACT_THRESHOLD = 18, FDX_ACT_LOG_SIGMOID = 19, FDX_ACT_HARD_TANH = 20, FDX_ACT_LOG = 21, FDX_ACT_COUNT = 22
};
typedef struct fdx_act {
    int kind;             /* FDX_ACT_*                                              */
    float max_value;
    float negative_slope;
    float threshold;
} fdx_act;

/* element-wise combinations of two operands with size-1 broadcasting (fdx_broadcast_combine_f32):
 * add_tensors / mult_tensors / subtract_tensors (include/fdeep/tensor.hpp:662-675), max_tensors / min_tensors
 * (:893-929), and PReLU's a > 0 ? a : b * a with b the learned slopes (layers/prelu_layer.hpp:29-70) */
enum { FDX_COMBINE_ADD = 0, FDX_COMBINE_MUL = 1, FDX_COMBINE_SUB = 2, FDX_COMBINE_MAX = 3, FDX_COMBINE_MIN = 4, FDX_COMBINE_PRELU = 5 };

const char* fdx_last_error(void);
/* lets a callback (custom layer) leave the text that fdx_last_error() reports for its failure */
void fdx_set_last_error(const char* text);
fdx_status fdx_init(int device);

/* ---- device memory plumbing for callers that do not link HIP themselves ---- */
fdx_status fdx_dev_alloc(size_t bytes, void** out);
fdx_status fdx_dev_free(void* p);
fdx_status fdx_h2d(void* dst_dev, const void* src_host, size_t bytes);
fdx_status fdx_d2h(void* dst_host, const void* src_dev, size_t bytes);
fdx_status fdx_sync(void);

/*
 * Conv2D, cross-correlation, implicit GEMM on fp32 MFMA:
 *   out[n][oy][ox][co] = act(bias[co] + sum_{fy,fx,ci} w[co][fy][fx][ci] * in[n][oy*sy+fy*dy-pad_top][ox*sx+fx*dx-pad_left][ci]
 *                            (+ residual[n][oy][ox][co]))
 * replaces convolve / convolve_accumulative (include/fdeep/convolution.hpp:398-429, 224-305).
 * Weights in the converted-JSON order [cout][kh][kw][cin] (keras_export/convert_model.py:197-200).
 * Out-of-range taps read zero, which is pad_tensor's zero fill (include/fdeep/tensor.hpp:490-517);
 * pad_top/pad_left and out_h/out_w come from fdx_window_geometry.
 * bias and residual may be NULL.
 */
fdx_status fdx_conv2d_nhwc_f32(const float* in, int n, int h, int w, int cin,
    const float* weights, const float* bias, int cout, int kh, int kw,
    int sy, int sx, int dy, int dx, int pad_top, int pad_left, int out_h, int out_w,
    const float* residual, const fdx_act* act, float* out);

/*
 * The same Conv2D for stem layers (1..4 input channels, square kernel, stride 2, dilation 1, cout a multiple of 4
 * and >= 64; fdx_conv2d_s2d_eligible says whether a layer qualifies): the input is first rewritten as its 2x2
 * space-to-depth image (into `scratch`, fdx_conv2d_s2d_scratch_bytes) so that a filter row reads one contiguous
 * run, then the implicit GEMM runs on that view.  weights_s2d comes from fdx_conv2d_s2d_prepare (host side, once
 * per layer, fdx_conv2d_s2d_weight_floats values).  Results equal fdx_conv2d_nhwc_f32 up to summation order.
 */
int fdx_conv2d_s2d_eligible(int cin, int kh, int kw, int sy, int sx, int dy, int dx, int cout);
size_t fdx_conv2d_s2d_scratch_bytes(int n, int out_h, int out_w, int cin, int k);
size_t fdx_conv2d_s2d_weight_floats(int cout, int cin, int k);
fdx_status fdx_conv2d_s2d_prepare(const float* weights, int cout, int cin, int k, float* weights_s2d);
fdx_status fdx_conv2d_s2d_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* weights_s2d,
    const float* bias, int cout, int k, int pad_top, int pad_left, int out_h, int out_w, const float* residual,
    const fdx_act* act, float* scratch, float* out);

/*
 * DepthwiseConv2D (depth multiplier 1); replaces depthwise_convolve
 * (include/fdeep/depthwise_convolution.hpp:21-99).  weights_hwc is [kh][kw][c]
 * (the converted-JSON slice_weights [c][kh][kw] transposed once at load).
 */
fdx_status fdx_dwconv2d_nhwc_f32(const float* in, int n, int h, int w, int c,
    const float* weights_hwc, const float* bias, int kh, int kw,
    int sy, int sx, int dy, int dx, int pad_top, int pad_left, int out_h, int out_w,
    const fdx_act* act, float* out);

/*
 * Depthwise 3x3 convolution (stride 1 or 2 in both directions, no dilation) followed by a 1x1 convolution, as one
 * launch whose intermediate tensor stays on the chip:
 *   mid[y][x][c]  = dw_act(dw_bias[c] + sum_taps dw_weights_hwc[fy][fx][c] * in[y*s - pad_top + fy][x*s - pad_left + fx][c])
 *   out[y][x][o]  = act(pw_bias[o] + sum_c pw_weights_nc[o][c] * mid[y][x][c] + residual[y][x][o])
 * replaces depthwise_convolve (include/fdeep/depthwise_convolution.hpp:21-99) followed by convolve with a 1x1 filter
 * (include/fdeep/convolution.hpp:398-429), the pair a SeparableConv2D is made of
 * (include/fdeep/layers/separable_conv_2d_layer.hpp:26-55) and the second half of an inverted-residual block
 * (DepthwiseConv2D, folded BatchNormalization, ReLU6, Conv2D 1x1).  Same results as the two launches up to the
 * summation order of the 1x1 product.  Needs c % 4 == 0, n_out <= 96, both activations NONE / RELU / GELU;
 * fdx_dwconv_pointwise_supported answers that without launching (FDX_ERR_UNSUPPORTED otherwise).
 */
int fdx_dwconv_pointwise_supported(int c, int n_out, int stride);
fdx_status fdx_dwconv_pointwise_nhwc_f32(const float* in, int n, int h, int w, int c, const float* dw_weights_hwc,
    const float* dw_bias, int stride, int pad_top, int pad_left, int out_h, int out_w, const fdx_act* dw_act,
    const float* pw_weights_nc, const float* pw_bias, int n_out, const float* residual, const fdx_act* act, float* out);

/*
 * A whole inverted-residual block as one launch: 1x1 convolution (expansion, cin -> ce) + activation, depthwise 3x3
 * (stride 1 or 2) + activation, 1x1 convolution (projection, ce -> n_out) + optional residual + activation; the expanded
 * tensor stays on chip (convolution.hpp:398-429, depthwise_convolution.hpp:21-99, convolution.hpp:398-429 run back to
 * back by the reference).  exp_weights_ec is [ce][cin], dw_weights_hwc [3][3][ce], pw_weights_nc [n_out][ce]; biases
 * may be NULL.  The padding (pad_top, pad_left; bottom / right implied by out_h, out_w) belongs to the depthwise
 * convolution and pads the expanded, activated tensor with zeros.  fdx_inverted_residual_supported tells whether the
 * kernel covers a shape: cin 16 / 24 / 32, ce % 4 == 0 within the LDS budget, n_out <= 64.
 */
int fdx_inverted_residual_supported(int cin, int ce, int n_out, int stride);
fdx_status fdx_inverted_residual_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* exp_weights_ec,
    const float* exp_bias, const fdx_act* exp_act, int ce, const float* dw_weights_hwc, const float* dw_bias, int stride, int pad_top,
    int pad_left, int out_h, int out_w, const fdx_act* dw_act, const float* pw_weights_nc, const float* pw_bias, int n_out,
    const float* residual, const fdx_act* act, float* out);

/*
 * 3x3 convolution, stride 1, no dilation, in the Winograd F(2x2, 3x3) form: 2.25 times fewer multiply-adds than the
 * direct sum that convolve runs (include/fdeep/convolution.hpp:398-429, :107-160); same result up to a few more
 * roundings (the transform matrices hold 0, +-1 and +-1/2 only).  The filter is moved into the transform domain once:
 * fdx_conv2d_winograd_prepare takes the converted-JSON order [cout][3][3][cin] (host memory) and writes
 * fdx_conv2d_winograd_weight_floats(cout, cin) floats (host memory), which the caller places on the device as
 * u_weights.  Needs cin % 8 == 0 and cout % 64 == 0 (fdx_conv2d_winograd_supported); zero padding pad_top / pad_left,
 * bottom / right implied by out_h / out_w as for fdx_conv2d_nhwc_f32.
 */
int fdx_conv2d_winograd_supported(int cin, int cout);
size_t fdx_conv2d_winograd_weight_floats(int cout, int cin);
fdx_status fdx_conv2d_winograd_prepare(const float* weights_nkkc, int cout, int cin, float* u_out);
fdx_status fdx_conv2d_winograd_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* u_weights, const float* bias,
    int cout, int pad_top, int pad_left, int out_h, int out_w, const float* residual, const fdx_act* act, float* out);

/*
 * The first block of a MobileNet-like network as one launch: a small convolution on the image (ek x ek taps on ic
 * channels with ek * ek * ic <= 32, e.g. 3x3 on RGB; stride conv_stride, zero padding conv_pad_top / conv_pad_left) +
 * activation, depthwise 3x3 (stride 1 or 2) + activation, 1x1 convolution (ce -> n_out) + optional residual +
 * activation.  The convolution's output (h x w x ce, the widest tensor of such a network) stays on chip; the reference
 * runs convolve (convolution.hpp:398-429), depthwise_convolve (depthwise_convolution.hpp:21-99) and convolve one
 * after the other.  conv_weights_nk is [ce][ek][ek][ic]; the other operands are those of
 * fdx_inverted_residual_nhwc_f32, (h, w) being the extents of the convolution's output, which the depthwise
 * convolution pads with zeros.  fdx_stem_block_supported tells whether the kernel covers a shape.
 */
int fdx_stem_block_supported(int ic, int ek, int ce, int n_out, int stride);
fdx_status fdx_stem_block_nhwc_f32(const float* in, int n, int ih, int iw, int ic, const float* conv_weights_nk,
    const float* conv_bias, const fdx_act* conv_act, int ce, int ek, int conv_stride, int conv_pad_top, int conv_pad_left, int h, int w,
    const float* dw_weights_hwc, const float* dw_bias, int stride, int pad_top, int pad_left, int out_h, int out_w, const fdx_act* dw_act,
    const float* pw_weights_nc, const float* pw_bias, int n_out, const float* residual, const fdx_act* act, float* out);

/*
 * Row-major GEMM with fused epilogue, fp32 MFMA:
 *   c[m][n] = act(alpha * sum_k a[m][k] * b_nk[n][k] + bias + residual[m][n])
 * replaces dense_layer::apply_impl (include/fdeep/layers/dense_layer.hpp:76-86; weights arrive
 * [in][out] and are transposed once at load to [out][in]) and dot_product_tensors
 * (include/fdeep/tensor.hpp:814-884).  bias_per_row selects bias[m] instead of bias[n].
 * batch > 1 runs `batch` independent problems; problem i uses
 *   a + (i / inner) * a_outer + (i % inner) * a_inner   (same for b, c); residual follows c.
 */
typedef struct fdx_gemm_batch {
    int batch, inner;
    int64_t a_outer, a_inner, b_outer, b_inner, c_outer, c_inner;
} fdx_gemm_batch;
fdx_status fdx_gemm_bias_act_f32(const float* a, int64_t lda, const float* b_nk, int64_t ldb,
    int m, int n, int k, float alpha, const float* bias, int bias_per_row,
    const float* residual, const fdx_act* act, float* c, int64_t ldc, const fdx_gemm_batch* batch);

/*
 * Dense on at most 16 rows (the decode shape): out[m][:] = act(x[m][:] * w_nk^T + bias + residual[m][:]),
 * an HBM-bound weight-streaming kernel (layers/dense_layer.hpp:76-86 at batch <= 16).
 */
fdx_status fdx_dense_rows_f32(const float* x, int m, int k, const float* w_nk, const float* bias, int n,
    const float* residual, const fdx_act* act, float* out);
/*
 * fdx_dense_rows_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arithmetic, same kernels and the
 * same results as fdx_dense_rows_f32; the split-K partial tiles and tickets it needs for k > 1024 live in a fixed
 * array of device memory inside the library (4 MiB + 16 KiB per GPU, held until the process ends) instead of a
 * workspace allocated on first use.  The call makes no hipMalloc / hipFree and uses no allocating library routine.
 * Needs fdx_init (or any earlier library call) to have run; limits: m <= 16, n <= 65536, k <= 32768 and
 * ceil(n / 16) * splits * 256 <= 1048576 floats (splits <= 8, chosen from k and n), otherwise FDX_ERR_INVALID with the
 * reason in fdx_last_error; an activation other than NONE / RELU / GELU answers FDX_ERR_UNSUPPORTED as in every launcher
 * with an epilogue.  One exception to "allocates nothing": while the per-kernel profile is switched on
 * (fdx_profile_enable, fdx_debug.h) every launch records two HIP events, which the runtime creates on first use; leave the
 * profile off where allocation is forbidden.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (other than in order on the library's stream) race.
 */
fdx_status fdx_dense_rows_noalloc_f32(const float* x, int m, int k, const float* w_nk, const float* bias, int n,
    const float* residual, const fdx_act* act, float* out);
/*
 * LayerNormalization followed by Dense in one launch (layers/layer_normalization_layer.hpp:37-63 then
 * layers/dense_layer.hpp:76-86).  fdx_fold_layernorm_f32 prepares, once per layer pair,
 *   w_folded[n][k] = w[n][k] * gamma[k],  w_rowsum[n] = sum_k w_folded[n][k],  bias_folded[n] = bias[n] + sum_k w[n][k] * beta[k]
 * (gamma / beta / bias may be NULL); the launch then computes rstd[m] * (x w_folded^T - mean[m] * w_rowsum) + bias_folded
 * with each row's mean and biased two-pass variance taken from x itself.  k <= 1024.
 */
fdx_status fdx_fold_layernorm_f32(const float* gamma, const float* beta, const float* w_nk, const float* bias, int n,
    int k, float* w_folded, float* w_rowsum, float* bias_folded);
fdx_status fdx_layernorm_dense_rows_f32(const float* x, int m, int k, float ln_eps, const float* w_folded,
    const float* w_rowsum, const float* bias_folded, int n, const float* residual, const fdx_act* act, float* out);

/* [rows][cols] -> [cols][rows] (load-time weight re-layout) */
fdx_status fdx_transpose_f32(const float* in, int rows, int cols, float* out);

/*
 * Max / average pooling with TF padding; mode 0 = max, 1 = average.  Window taps outside
 * [0,h)x[0,w) are ignored by max and excluded from the average's divisor
 * (include/fdeep/layers/max_pooling_3d_layer.hpp:17-38, average_pooling_3d_layer.hpp:17-42).
 * zero_top/left/bottom/right describe an explicit ZeroPadding2D folded into this call: taps in
 * that frame (still outside the stored tensor) contribute the value 0 and count as real elements.
 */
fdx_status fdx_pool2d_nhwc_f32(const float* in, int n, int h, int w, int c, int ph, int pw, int sy, int sx,
    int pad_top, int pad_left, int zero_top, int zero_left, int zero_bottom, int zero_right,
    int out_h, int out_w, int mode, float* out);

/* global max (mode 0) / average (mode 1) over all positions of each sample:
 * include/fdeep/layers/global_average_pooling_3d_layer.hpp:25-41 */
fdx_status fdx_global_pool_f32(const float* in, int n, int positions, int c, int mode, float* out);

/* out = act(a + b), b broadcast if b_count < count (b_count divides count; trailing dims match):
 * add_layer / sum_tensors, include/fdeep/tensor.hpp:642-680 */
fdx_status fdx_eltwise_add_f32(const float* a, const float* b, size_t count, size_t b_count,
    const fdx_act* act, float* out);
/* out = act(x) ; relu family and erf-GELU (include/fdeep/layers/relu_layer.hpp:32-48,
 * include/fdeep/recurrent_ops.hpp:73-76) */
fdx_status fdx_activation_f32(const float* x, size_t count, const fdx_act* act, float* out);
/* out = act(x * scale[c] + shift[c]) along the last axis: a BatchNormalization that could not be
 * folded into its producer (include/fdeep/tensor.hpp:773-793) */
fdx_status fdx_channel_affine_f32(const float* x, size_t positions, int c, const float* scale,
    const float* shift, const fdx_act* act, float* out);
/* explicit zero padding, zero_padding_3d_layer / pad_tensor (include/fdeep/tensor.hpp:490-517) */
fdx_status fdx_zero_pad2d_nhwc_f32(const float* in, int n, int h, int w, int c, int pt, int pb, int pl, int pr,
    float* out);

/* LayerNormalization over the last `depth` elements of each row
 * (include/fdeep/layers/layer_normalization_layer.hpp:37-63, tensor.hpp:758-793); gamma/beta may be NULL */
fdx_status fdx_layernorm_f32(const float* x, int64_t rows, int depth, const float* gamma, const float* beta,
    float eps, float* out);
/* LayerNormalization over any subset of the five right-aligned axes of each sample
 * (layer_normalization_layer.hpp:37-61: moments over `axes`, gamma / beta shaped like the normalised
 * axes).  dims5 = (dim5, dim4, height, width, depth); bit i of axes_mask selects dims5[i]; gamma / beta
 * hold one value per position on the selected axes, in storage order.  Trailing axes take the
 * row kernel above. */
fdx_status fdx_layernorm_axes_f32(const float* x, int batch, const int64_t* dims5, unsigned axes_mask, const float* gamma,
    const float* beta, float eps, float* out);
/* RMSNormalization over the selected axes: x / sqrt(mean(x^2) + eps) * scale
 * (include/fdeep/layers/rms_normalization_layer.hpp:37-69); arguments as fdx_layernorm_axes_f32 */
fdx_status fdx_rmsnorm_axes_f32(const float* x, int batch, const int64_t* dims5, unsigned axes_mask, const float* scale,
    float eps, float* out);
/* out = act(a + b) with size-1 broadcasting on any of the five right-aligned axes, per sample
 * (elem_wise_combine_tensors, include/fdeep/tensor.hpp:642-660); `batch` samples of each operand lie
 * back to back; out_dims5 (may be NULL) receives the per-axis maximum */
fdx_status fdx_broadcast_add_f32(const float* a, const int64_t* a_dims5, const float* b, const int64_t* b_dims5,
    int batch, const fdx_act* act, float* out, int64_t* out_dims5);
/* the same with any FDX_COMBINE_* operation, then out = act(scale * combine(a, b)) (scale serves
 * average_tensors, tensor.hpp:886-891); b_shared != 0: one b for all samples (learned parameters) */
fdx_status fdx_broadcast_combine_f32(int op, const float* a, const int64_t* a_dims5, const float* b, const int64_t* b_dims5,
    int b_shared, int batch, float scale, const fdx_act* act, float* out, int64_t* out_dims5);
/* Concatenate along one axis (concatenate_tensors, include/fdeep/tensor.hpp:459-483): input i is
 * `outer` rows of inner[i] floats (inner = extent on the axis times everything to its right, outer =
 * batch times everything to its left); rows are laid side by side in `out` */
fdx_status fdx_concat_f32(const float* const* ins, int n_inputs, const int64_t* inner, int64_t outer, float* out);
/* Permute (permute_tensor, include/fdeep/tensor.hpp:526-549): output axis i of each sample is input axis perm[i]
 * (0-based; the layer's `dims` minus one); dims = the sample's `rank` extents */
fdx_status fdx_permute_f32(const float* in, int batch, int rank, const int64_t* dims, const int* perm, float* out);
/* Cropping1D / Cropping2D (crop_tensor, include/fdeep/tensor.hpp:586-610) */
fdx_status fdx_crop2d_nhwc_f32(const float* in, int n, int h, int w, int c, int top, int bottom, int left, int right, float* out);
/* Zero insertion in front of a transposed convolution (dilate_tensor, include/fdeep/tensor.hpp:612-640, called by
 * convolve_transposed, include/fdeep/convolution.hpp:443-469): the output has (h-1)*rate_y+1 by (w-1)*rate_x+1 pixels,
 * plus rate-1 more with the larger half in front when trailing_zeros is set (the layer's "same" padding) and the
 * rate is not (1, 1).  Conv2DTranspose = this, then fdx_conv2d_nhwc_f32 with stride 1 on the mirrored filter. */
fdx_status fdx_dilate2d_nhwc_f32(const float* in, int n, int h, int w, int c, int rate_y, int rate_x, int trailing_zeros,
    float* out);
/* UpSampling1D / UpSampling2D by integer factors, nearest or bilinear (resize2d_nearest / resize2d_bilinear,
 * include/fdeep/tensor.hpp:959-974, 997-1035; layers/upsampling_2d_layer.hpp) */
fdx_status fdx_upsample2d_nhwc_f32(const float* in, int n, int h, int w, int c, int factor_y, int factor_x, int bilinear,
    float* out);
/* EinsumDense, any equation "lhs,kernel->rhs" the reference evaluates
 * (include/fdeep/layers/einsum_dense_layer.hpp:125-258): in_dims are the extents of the trailing
 * in_rank characters of lhs (missing leading ones count as 1; with a batch the first lhs character
 * simply has extent `batch`), kernel_dims those of the kernel as stored in the file, bias (NULL when
 * bias_axes is NULL or empty) is laid out over the bias axes in rhs order (:197-222),
 * full_output_shape (may be NULL) gives one extent per rhs character for characters that occur only
 * in the output.  The output keeps every rhs character, the leading one included; out_rank /
 * out_dims (up to 6 entries, may be NULL) receive its shape. */
fdx_status fdx_einsum_dense_f32(const char* equation, const char* bias_axes, const float* in, int in_rank,
    const int64_t* in_dims, const float* kernel, int kernel_rank, const int64_t* kernel_dims, const float* bias,
    const int64_t* full_output_shape, const fdx_act* act, float* out, int* out_rank, int64_t* out_dims);
/* softmax over the last axis in the reference's exp(x - m - log(sum)) form (tensor.hpp:1165-1192);
 * causal_period > 0 masks row r to its first (r % causal_period) + 1 + causal_offset entries
 * (the prefix identity of causal self-attention; no counterpart in the reference, which has no mask) */
fdx_status fdx_softmax_f32(const float* x, int64_t rows, int depth, int causal_period, int causal_offset,
    float* out);
/* rows of `table` selected by float ids truncated to size_t (include/fdeep/layers/embedding_layer.hpp:38-58).
 * error_flag_dev (may be NULL) is set to 1 on the device if an id is out of range. */
fdx_status fdx_embedding_f32(const float* ids, int64_t count, const float* table, int input_dim, int output_dim,
    float* out, int* error_flag_dev);
/* first maximum of each row (tensor_max_pos, include/fdeep/tensor.hpp:281-302) */
fdx_status fdx_argmax_f32(const float* x, int64_t rows, int depth, int32_t* out_idx, float* out_val);

/*
 * MultiHeadAttention core for already projected q/k/v (prefill shape):
 *   out[b][t][h][:] = softmax_s(scale * q[b][t][h] . k[b][s][h]) * v[b][s][h]
 * q [b][t][heads*dk], k [b][s][heads*dk], v [b][s][heads*dv], out [b][t][heads*dv]
 * (apply_head, include/fdeep/layers/multi_head_attention_layer.hpp:74-95).  causal != 0 lets query t
 * see keys 0..t+(s-t_len) only.  scratch_dev must hold fdx_mha_scratch_bytes().
 */
size_t fdx_mha_scratch_bytes(int batch, int heads, int t, int s, int dv);
fdx_status fdx_mha_prefill_f32(const float* q, const float* k, const float* v, int batch, int t, int s,
    int heads, int dk, int dv, int causal, float* out, void* scratch_dev);
/*
 * Decode step: one query row per sequence against a key/value cache.
 * q [b][heads*dk]; k_cache [b][max_len][heads*dk], v_cache [b][max_len][heads*dv] (token-major, so the
 * projection GEMM of a new token writes its row in place); len = keys visible (incl. the newest).
 */
fdx_status fdx_mha_decode_f32(const float* q, const float* k_cache, const float* v_cache, int batch, int heads,
    int dk, int dv, int len, int max_len, float* out);

/* TF window geometry shared by conv and pooling (include/fdeep/convolution.hpp:320-396):
 * padding 0 valid, 1 same, 2 causal; geom = pad_top, pad_bottom, pad_left, pad_right, out_h, out_w */
fdx_status fdx_window_geometry(int in_h, int in_w, int k_h, int k_w, int s_h, int s_w, int padding, int* geom);

/* ---------------------------------------------------------------- whole models */
typedef struct fdx_model fdx_model;
typedef struct fdx_session fdx_session;

/*
 * Parses a converted-JSON model (the output format of keras_export/convert_model.py:971-1001),
 * uploads the weights once (they stay resident in HBM) and builds the launch plan.
 * Replaces read_model (include/fdeep/model.hpp:198-281).  verify != 0 replays the file's embedded
 * test cases with absolute tolerance verify_epsilon (model.hpp:254-267, import_model.hpp:1990-2021).
 */
fdx_status fdx_model_create(const char* json, size_t len, int verify, float verify_epsilon, fdx_model** out);
/*
 * The host half of fdx_model_create alone, for machines without a GPU: what read_model does to a file before the first
 * prediction (include/fdeep/model.hpp:198-253, import_model.hpp:274-297 for the parameter arrays): parses the text, builds the
 * layer graph, decodes every parameter array and embedded test tensor and infers all shapes, with unknown extents set to
 * unknown_extent (> 0).  Returns the status and message fdx_model_create would give for the same defect; touches no device.
 * Files that need a custom layer creator answer FDX_ERR_UNSUPPORTED here.
 */
fdx_status fdx_model_check(const char* json, size_t len, int64_t unknown_extent);
/* ---- host fallback for layer classes the device path does not implement ----
 * The counterpart of the reference's extension point: internal::layer_creators, a map from class name
 * to a factory of layer objects whose apply_impl runs on host tensors
 * (include/fdeep/import_model.hpp:374-381, 1944-1950; include/fdeep/layers/layer.hpp:32-88).  A class
 * registered here takes precedence over a built-in one, as in the reference's map_union.  The layer
 * runs on the host, one sample at a time, between device segments: the stream is drained, the inputs
 * are copied to host memory, `apply` is called per sample, and the output is copied back. */
typedef fdx_status (*fdx_param_getter)(void* ctx, const char* layer_name, const char* param_name,
    const float** values, size_t* count); /* decoded trainable_params entry; valid until `create` returns */
typedef struct fdx_custom_layer {
    const char* class_name;
    /* once per layer of this class while the model is built; config_json is the layer's JSON object */
    fdx_status (*create)(void* user, const char* layer_name, const char* config_json, size_t config_len,
        fdx_param_getter get_param, void* get_param_ctx, void** instance);
    /* one sample: n_inputs host tensors, each with a rank and five right-aligned extents; writes the output's
     * rank and extents, and its values unless `output` is NULL (the shape pass at plan time) */
    fdx_status (*apply)(void* instance, int n_inputs, const float* const* inputs, const int* in_ranks,
        const int64_t* in_dims5, float* output, int* out_rank, int64_t* out_dims5);
    void (*destroy)(void* instance);
    void* user;
} fdx_custom_layer;
/* fdx_model_create with custom layers (load_model's custom_layer_creators argument, model.hpp:285-301) */
fdx_status fdx_model_create_custom(const char* json_text, size_t len, int verify, float verify_epsilon,
    const fdx_custom_layer* custom_layers, int n_custom_layers, fdx_model** out);
fdx_status fdx_model_destroy(fdx_model* m);
fdx_status fdx_model_name(const fdx_model* m, const char** name, const char** hash);
/* number of inputs/outputs and their shapes: rank and dims (-1 = variable), model.hpp:66-96 */
fdx_status fdx_model_io_count(const fdx_model* m, int* n_inputs, int* n_outputs);
fdx_status fdx_model_io_shape(const fdx_model* m, int is_output, int index, int* rank, int64_t* dims5);
/*
 * predict / predict_multi (include/fdeep/model.hpp:23-42,132-151): `batch` independent samples in one
 * launch sequence.  in[i] points at batch * volume(in_dims[i]) floats (sample-major); in_dims holds
 * 5 right-aligned dims per input and in_ranks its rank (the reference rejects a rank mismatch,
 * tensor_shape.hpp:246-250).  Outputs: out[i] receives batch * volume floats; out_dims/out_ranks are
 * written per output.  Host-pointer and device-pointer variants.  The device-pointer variant returns with its work
 * queued on the library's stream (fdx_sync waits for it) and reads inputs that are 16-byte aligned where they lie
 * (others are copied first): such an input must stay unchanged until that work has completed.
 */
fdx_status fdx_model_predict(fdx_model* m, int batch, const float* const* in, const int64_t* in_dims,
    const int* in_ranks, float* const* out, int64_t* out_dims, int* out_ranks);
/* fdx_model_predict with every input given as `batch` pointers to single samples, in_samples[i * batch + b] = sample b of
 * input i: the form predict_multi receives its tensors in (include/fdeep/model.hpp:28-42), so that a caller who holds
 * one buffer per sample does not have to concatenate them first.  Host pointers; returns after the outputs are written. */
fdx_status fdx_model_predict_samples(fdx_model* m, int batch, const float* const* in_samples, const int64_t* in_dims,
    const int* in_ranks, float* const* out, int64_t* out_dims, int* out_ranks);
fdx_status fdx_model_predict_dev(fdx_model* m, int batch, const float* const* in_dev, const int64_t* in_dims,
    const int* in_ranks, float* const* out_dev, int64_t* out_dims, int* out_ranks);
/* output shapes for given input shapes without running anything */
fdx_status fdx_model_infer_shapes(fdx_model* m, const int64_t* in_dims, const int* in_ranks, int64_t* out_dims,
    int* out_ranks);
/* 2 * multiply-accumulates of the Conv2D/Dense/attention contractions of the last planned batch */
fdx_status fdx_model_last_flops(const fdx_model* m, double* flops);

/*
 * Autoregressive session over a decoder model with inputs (ids, positions) and one logits output:
 * causal self-attention with projected keys/values cached in HBM.  The reference has neither a mask
 * nor a cache (layers/multi_head_attention_layer.hpp:74-95); position t of a session equals the
 * reference's MultiHeadAttention(query = x[t:t+1], value = x[0:t+1]) (same file, :98-103).
 * prefill consumes `t` ids per sequence ([batch][t], float), decode_step one id per sequence.
 * logits_dev (may be NULL) receives [batch][vocab] of the last position; next_ids_dev (may be NULL)
 * the greedy argmax as floats (first maximum wins, tensor.hpp:281-302).
 */
fdx_status fdx_session_create(fdx_model* m, int batch, int max_len, fdx_session** out);
fdx_status fdx_session_destroy(fdx_session* s);
fdx_status fdx_session_reset(fdx_session* s);
fdx_status fdx_session_prefill(fdx_session* s, const float* ids_dev, int t, float* logits_dev, float* next_ids_dev);
fdx_status fdx_session_decode_step(fdx_session* s, const float* ids_dev, float* logits_dev, float* next_ids_dev);
/* runs `steps` greedy decode steps feeding each step's argmax back in; tokens_dev gets [steps][batch] floats */
fdx_status fdx_session_decode_greedy(fdx_session* s, const float* first_ids_dev, int steps, float* tokens_dev,
    float* last_logits_dev);
fdx_status fdx_session_length(const fdx_session* s, int* len);

/*
 * The per-shape tuning table (no counterpart in the reference).  By default nothing is timed: every kernel choice
 * (tile, K cut, direct against Winograd convolution, the form of a depthwise block) follows closed rules, the same in
 * every process, and the first predict of a shape costs what any later one costs plus plan building.
 * fdx_tuner_timing(1) (or FDX_AUTOTUNE=1 in the environment) lets the first launch of a convolution / GEMM shape (and of
 * a depthwise 3x3 + 1x1 pair) time the candidate kernels once per process and keep the winner: about a second for a
 * ResNet50 at batch 64, for 0-2 % more throughput.  Candidates sum in different orders, so two processes that time may
 * return results that differ in the last bits (all within the reference tolerance; the reference itself leaves the
 * summation order to Eigen, convolution.hpp:134-148).  A deployment that wants the timed choices without timing exports
 * the table of a warmed-up process, imports it at start-up and freezes it: a listed shape takes its row, an unlisted one
 * the closed rule.  Text format: one line per shape, "conv M N K Cin kh kw sy sx batch res choice".
 * fdx_tuner_export: `needed` receives the size including the terminator; text may be NULL to query it.
 */
fdx_status fdx_tuner_timing(int on);
fdx_status fdx_tuner_export(char* text, size_t capacity, size_t* needed);
fdx_status fdx_tuner_import(const char* text);
fdx_status fdx_tuner_freeze(int on);

#ifdef __cplusplus
}
#endif
#endif
