/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C, single-threaded, fp32 restatement of the per-layer forward
 * functions that frugally-deep's fdeep::model::predict runs on the CPU.
 * It exists to check the HIP path and to be timed as the "port" CPU
 * baseline.  Only tests, the smoke check and the bench's cpu_baseline leg
 * may load it; the product library never does.
 *
 * All tensors are channels-last fp32, one sample per call (the reference
 * has no batch dimension, include/fdeep/tensor_shape.hpp:26-28).
 *
 * Every function cites the reference lines (relative to the reference
 * checkout) whose arithmetic it follows.  The genuine reference cannot be
 * compiled here (its headers need Eigen, FunctionalPlus and nlohmann/json,
 * none of which is installed), so each function is pinned by independent
 * checks in tests/test_oracle_*.py: brute-force definitions, fp64 library
 * routines (numpy / scipy / torch CPU) and closed forms.
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FDO_PAD_VALID 0
#define FDO_PAD_SAME 1
#define FDO_PAD_CAUSAL 2

/* fplus::ceil(x - 0.001) on a float quotient, include/fdeep/convolution.hpp:339-348 */
static int ceil_fudge(int num, int den)
{
    double v = (double)((float)num / (float)den) - 0.001;
    return (int)ceil(v);
}

/*
 * Output size and TF-style padding of a 2-D window op.
 * include/fdeep/convolution.hpp:320-396 (preprocess_convolution, transposed == false)
 * and include/fdeep/convolution3d.hpp:35-134 for pooling (same rules per axis).
 * k_h / k_w are the *effective* (dilated) sizes, convolution.hpp:408-414.
 * geom = { pad_top, pad_bottom, pad_left, pad_right, out_h, out_w }
 */
int fdo_window_geometry(int in_h, int in_w, int k_h, int k_w, int s_h, int s_w,
    int pad_type, int* geom)
{
    int out_h, out_w, pt = 0, pb = 0, pl = 0, pr = 0;
    if (pad_type == FDO_PAD_SAME || pad_type == FDO_PAD_CAUSAL) {
        out_h = ceil_fudge(in_h, s_h);
        out_w = ceil_fudge(in_w, s_w);
    } else {
        out_h = ceil_fudge(in_h - k_h + 1, s_h);
        out_w = ceil_fudge(in_w - k_w + 1, s_w);
    }
    if (pad_type == FDO_PAD_SAME) {
        int along_h, along_w;
        if (in_h % s_h == 0)
            along_h = k_h - s_h > 0 ? k_h - s_h : 0;
        else
            along_h = k_h - (in_h % s_h) > 0 ? k_h - (in_h % s_h) : 0;
        if (in_w % s_w == 0)
            along_w = k_w - s_w > 0 ? k_w - s_w : 0;
        else
            along_w = k_w - (in_w % s_w) > 0 ? k_w - (in_w % s_w) : 0;
        pt = along_h / 2;
        pb = along_h - pt;
        pl = along_w / 2;
        pr = along_w - pl;
    } else if (pad_type == FDO_PAD_CAUSAL) {
        pt = k_h - 1;
        pl = k_w - 1;
    }
    if (out_h < 0 || out_w < 0)
        return -1; /* integral_cast_throw, convolution.hpp:386-391 */
    geom[0] = pt; geom[1] = pb; geom[2] = pl; geom[3] = pr;
    geom[4] = out_h; geom[5] = out_w;
    return 0;
}

/* pad_tensor, include/fdeep/tensor.hpp:490-517 (2-D part) */
void fdo_pad2d(const float* in, int h, int w, int c, int pt, int pb, int pl, int pr,
    float value, float* out)
{
    const int oh = h + pt + pb, ow = w + pl + pr;
    for (size_t i = 0; i < (size_t)oh * ow * c; ++i)
        out[i] = value;
    for (int y = 0; y < h; ++y)
        memcpy(out + ((size_t)(y + pt) * ow + pl) * c, in + (size_t)y * w * c,
            sizeof(float) * (size_t)w * c);
}

/* C[M x N] += A[M x K] (row stride lda) * B[K x N] (row stride ldb); C row stride ldc.
 * Stands in for Eigen's `noalias() += A * B` (include/fdeep/convolution.hpp:147,274). */
static void sgemm_acc(int M, int N, int K, const float* A, size_t lda,
    const float* B, size_t ldb, float* C, size_t ldc)
{
    int m = 0;
    for (; m + 4 <= M; m += 4) {
        const float* a0 = A + (size_t)m * lda;
        const float* a1 = a0 + lda;
        const float* a2 = a1 + lda;
        const float* a3 = a2 + lda;
        float* c0 = C + (size_t)m * ldc;
        float* c1 = c0 + ldc;
        float* c2 = c1 + ldc;
        float* c3 = c2 + ldc;
        for (int k = 0; k < K; ++k) {
            const float* b = B + (size_t)k * ldb;
            const float x0 = a0[k], x1 = a1[k], x2 = a2[k], x3 = a3[k];
            for (int n = 0; n < N; ++n) {
                const float bv = b[n];
                c0[n] += x0 * bv;
                c1[n] += x1 * bv;
                c2[n] += x2 * bv;
                c3[n] += x3 * bv;
            }
        }
    }
    for (; m < M; ++m) {
        const float* a0 = A + (size_t)m * lda;
        float* c0 = C + (size_t)m * ldc;
        for (int k = 0; k < K; ++k) {
            const float* b = B + (size_t)k * ldb;
            const float x0 = a0[k];
            for (int n = 0; n < N; ++n)
                c0[n] += x0 * b[n];
        }
    }
}

/*
 * Load-time filter re-layout: converted-JSON order [Cout][kh][kw][Cin]
 * (keras_export/convert_model.py:197-200) to [kh][kw][Cin][Cout]
 * (include/fdeep/filter.hpp:69-103, include/fdeep/convolution.hpp:29-60).
 */
void fdo_conv2d_prepare(const float* w_json, int cout, int kh, int kw, int cin, float* w_hwio)
{
    for (int n = 0; n < cout; ++n)
        for (int y = 0; y < kh; ++y)
            for (int x = 0; x < kw; ++x)
                for (int z = 0; z < cin; ++z)
                    w_hwio[(((size_t)y * kw + x) * cin + z) * cout + n] =
                        w_json[(((size_t)n * kh + y) * kw + x) * cin + z];
}

/*
 * Conv2D forward on an already padded input: output initialised to the bias,
 * then one accumulating GEMM per filter row (per filter tap when the x
 * dilation breaks contiguity), input windows overlapped by their row stride
 * instead of an im2col copy.
 * include/fdeep/convolution.hpp:62-84 (init to bias), 224-305 (convolve_accumulative),
 * 86-103 (overlapping-window mapping), 107-222 (stride-1 / dilated variants compute
 * the same sums).
 */
void fdo_conv2d_padded(const float* inp, int ph, int pw, int cin,
    const float* w_hwio, const float* bias, int cout, int kh, int kw,
    int sy, int sx, int dy, int dx, int out_h, int out_w, float* out)
{
    (void)ph;
    for (size_t p = 0; p < (size_t)out_h * out_w; ++p)
        for (int n = 0; n < cout; ++n)
            out[p * cout + n] = bias ? bias[n] : 0.0f;
    for (int yf = 0; yf < kh; ++yf) {
        for (int y = 0; y < out_h; ++y) {
            const float* in_row = inp + (size_t)(y * sy + yf * dy) * pw * cin;
            float* out_row = out + (size_t)y * out_w * cout;
            if (dx == 1) {
                sgemm_acc(out_w, cout, kw * cin, in_row, (size_t)sx * cin,
                    w_hwio + (size_t)yf * kw * cin * cout, (size_t)cout, out_row, (size_t)cout);
            } else {
                for (int xf = 0; xf < kw; ++xf)
                    sgemm_acc(out_w, cout, cin, in_row + (size_t)xf * dx * cin, (size_t)sx * cin,
                        w_hwio + ((size_t)yf * kw + xf) * cin * cout, (size_t)cout, out_row,
                        (size_t)cout);
            }
        }
    }
}

/*
 * Conv2D layer: geometry, padded copy, accumulate.
 * include/fdeep/convolution.hpp:398-429 (convolve), layers/conv_2d_layer.hpp:44-48.
 * Returns 0 and fills out_hw = {out_h, out_w}; out must hold out_h*out_w*cout floats
 * (call with out == NULL to query the size only).
 */
int fdo_conv2d(const float* in, int h, int w, int cin, const float* w_hwio, const float* bias,
    int cout, int kh, int kw, int sy, int sx, int dy, int dx, int pad_type,
    float* out, int* out_hw)
{
    int g[6];
    const int ekh = (kh - 1) * dy + 1, ekw = (kw - 1) * dx + 1;
    if (fdo_window_geometry(h, w, ekh, ekw, sy, sx, pad_type, g) != 0)
        return -1;
    out_hw[0] = g[4];
    out_hw[1] = g[5];
    if (!out)
        return 0;
    const int ph = h + g[0] + g[1], pw = w + g[2] + g[3];
    float* padded = (float*)malloc(sizeof(float) * (size_t)ph * pw * cin);
    if (!padded)
        return -2;
    fdo_pad2d(in, h, w, cin, g[0], g[1], g[2], g[3], 0.0f, padded);
    fdo_conv2d_padded(padded, ph, pw, cin, w_hwio, bias, cout, kh, kw, sy, sx, dy, dx, g[4], g[5], out);
    free(padded);
    return 0;
}

/*
 * Conv2DTranspose / Conv1DTranspose layer.  The filter arrives in the converted-JSON order
 * [Cout][kh][kw][Cin] (keras_export/convert_model.py:221-224) and is mirrored in height and
 * width at load (include/fdeep/filter.hpp:94-97); w_hwio_flipped is that mirrored filter in
 * [kh][kw][Cin][Cout] order (fdo_conv2d_prepare of the mirrored array).  Forward
 * (include/fdeep/convolution.hpp:443-469): zeros are inserted between the input pixels
 * (dilate_tensor, include/fdeep/tensor.hpp:612-640 -- with "same" padding sy-1 / sx-1
 * further zeros are added, the larger half in front), the result is padded by the
 * transposed branch of preprocess_convolution (convolution.hpp:320-396: kh-1 / kw-1 on every
 * side for "valid", the stride-1 "same" split otherwise) and convolved with stride 1.
 * Filter dilation is applied to the filter before mirroring (filter.hpp:93), so (dy, dx) act
 * as an ordinary dilation of the mirrored filter and the window uses the inflated size.
 * "causal" fails the reference's own output-width assertion (convolution.hpp:243) for any
 * filter wider than one tap and is rejected here.
 */
int fdo_conv2d_transpose(const float* in, int h, int w, int cin, const float* w_hwio_flipped, const float* bias,
    int cout, int kh, int kw, int sy, int sx, int dy, int dx, int pad_type,
    float* out, int* out_hw)
{
    if (pad_type != 0 && pad_type != 1)
        return -1;
    const int same = pad_type == 1;
    const int ekh = (kh - 1) * dy + 1, ekw = (kw - 1) * dx + 1;
    const int exp_y = (same && !(sy == 1 && sx == 1)) ? sy - 1 : 0;
    const int exp_x = (same && !(sy == 1 && sx == 1)) ? sx - 1 : 0;
    const int dh = (h - 1) * sy + 1 + exp_y, dw = (w - 1) * sx + 1 + exp_x;
    const int off_y = exp_y - exp_y / 2, off_x = exp_x - exp_x / 2;
    int pt, pb, pl, pr, oh, ow;
    if (same) {
        /* stride 1: in % 1 == 0 -> pad_along = max(filter - 1, 0) */
        oh = dh;
        ow = dw;
        pt = (ekh - 1) / 2; pb = (ekh - 1) - pt;
        pl = (ekw - 1) / 2; pr = (ekw - 1) - pl;
    } else {
        oh = dh + ekh - 1;
        ow = dw + ekw - 1;
        pt = pb = ekh - 1;
        pl = pr = ekw - 1;
    }
    out_hw[0] = oh;
    out_hw[1] = ow;
    if (!out)
        return 0;
    const int ph = dh + pt + pb, pw = dw + pl + pr;
    float* padded = (float*)calloc((size_t)ph * pw * cin, sizeof(float));
    if (!padded)
        return -2;
    for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
            memcpy(padded + ((size_t)(y * sy + off_y + pt) * pw + (x * sx + off_x + pl)) * cin,
                in + ((size_t)y * w + x) * cin, sizeof(float) * (size_t)cin);
    fdo_conv2d_padded(padded, ph, pw, cin, w_hwio_flipped, bias, cout, kh, kw, 1, 1, dy, dx, oh, ow, out);
    free(padded);
    return 0;
}

/*
 * DepthwiseConv2D (depth multiplier 1).  Filter arrives in converted-JSON order
 * [C][kh][kw] (keras_export/convert_model.py:203-206) and is inflated with zeros
 * for dilation at load (include/fdeep/filter.hpp:93,
 * layers/depthwise_conv_2d_layer.hpp:28-48); the window then uses the inflated size.
 * Accumulation: include/fdeep/depthwise_convolution.hpp:21-72 (bias first, then per
 * filter row, per output pixel, sum over the row's taps).
 */
int fdo_depthwise_conv2d(const float* in, int h, int w, int c, const float* w_json,
    const float* bias, int kh, int kw, int sy, int sx, int dy, int dx, int pad_type,
    float* out, int* out_hw)
{
    int g[6];
    const int ekh = (kh - 1) * dy + 1, ekw = (kw - 1) * dx + 1;
    if (fdo_window_geometry(h, w, ekh, ekw, sy, sx, pad_type, g) != 0)
        return -1;
    out_hw[0] = g[4];
    out_hw[1] = g[5];
    if (!out)
        return 0;
    const int ph = h + g[0] + g[1], pw = w + g[2] + g[3];
    float* padded = (float*)malloc(sizeof(float) * (size_t)ph * pw * c);
    float* filt = (float*)calloc((size_t)ekh * ekw * c, sizeof(float));
    if (!padded || !filt) {
        free(padded);
        free(filt);
        return -2;
    }
    for (int z = 0; z < c; ++z)
        for (int y = 0; y < kh; ++y)
            for (int x = 0; x < kw; ++x)
                filt[((size_t)(y * dy) * ekw + x * dx) * c + z] = w_json[((size_t)z * kh + y) * kw + x];
    fdo_pad2d(in, h, w, c, g[0], g[1], g[2], g[3], 0.0f, padded);
    const int out_h = g[4], out_w = g[5];
    for (size_t p = 0; p < (size_t)out_h * out_w; ++p)
        for (int z = 0; z < c; ++z)
            out[p * c + z] = bias ? bias[z] : 0.0f;
    for (int yf = 0; yf < ekh; ++yf) {
        const float* frow = filt + (size_t)yf * ekw * c;
        for (int y = 0; y < out_h; ++y) {
            const float* in_row = padded + (size_t)(y * sy + yf) * pw * c;
            for (int x = 0; x < out_w; ++x) {
                const float* win = in_row + (size_t)x * sx * c;
                float* o = out + ((size_t)y * out_w + x) * c;
                for (int z = 0; z < c; ++z) {
                    float s = 0.0f;
                    for (int xf = 0; xf < ekw; ++xf)
                        s += win[(size_t)xf * c + z] * frow[(size_t)xf * c + z];
                    o[z] += s;
                }
            }
        }
    }
    free(padded);
    free(filt);
    return 0;
}

/*
 * Dense: every last-axis row r gets y[r] = x[r] * W + b, one vector-matrix product
 * per row, W in converted-JSON order [in][out].
 * include/fdeep/layers/dense_layer.hpp:22-101 (bias stored as an extra weight row, 24-30;
 * per-row product 76-86).
 */
void fdo_dense(const float* x, int rows, int n_in, const float* w, const float* bias,
    int n_out, float* y)
{
    for (int r = 0; r < rows; ++r) {
        float* yr = y + (size_t)r * n_out;
        for (int n = 0; n < n_out; ++n)
            yr[n] = 0.0f;
        sgemm_acc(1, n_out, n_in, x + (size_t)r * n_in, (size_t)n_in, w, (size_t)n_out, yr,
            (size_t)n_out);
        if (bias)
            for (int n = 0; n < n_out; ++n)
                yr[n] += bias[n]; /* last row of the augmented matrix times the appended 1 */
    }
}

/*
 * Softmax along depth for each row: max, sum of exp(x-m), exp(x - m - log(sum)),
 * infinities mapped to 0.  include/fdeep/tensor.hpp:1165-1192.
 */
void fdo_softmax(const float* x, int rows, int depth, float* y)
{
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * depth;
        float* yr = y + (size_t)r * depth;
        float m = -FLT_MAX;
        for (int z = 0; z < depth; ++z)
            m = xr[z] > m ? xr[z] : m;
        float s = 0.0f;
        for (int z = 0; z < depth; ++z)
            s += expf(xr[z] - m);
        const float ls = logf(s);
        for (int z = 0; z < depth; ++z) {
            const float v = expf(xr[z] - m - ls);
            yr[z] = isinf(v) ? 0.0f : v;
        }
    }
}

/*
 * LayerNormalization over the trailing `depth` elements of each row:
 * mean, biased two-pass variance (sum of |x-mean|^2 / n), then
 * x*inv + (beta - mean*inv) with inv = gamma / sqrt(var + eps).
 * include/fdeep/layers/layer_normalization_layer.hpp:37-63,
 * include/fdeep/tensor.hpp:758-771 (moments), 773-793 (batch_normalization).
 * gamma / beta may be NULL (treated as 1 / 0, layer_normalization_layer.hpp:60-61).
 */
void fdo_layernorm(const float* x, int rows, int depth, const float* gamma, const float* beta,
    float eps, float* y)
{
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * depth;
        float* yr = y + (size_t)r * depth;
        float sum = 0.0f;
        for (int z = 0; z < depth; ++z)
            sum += xr[z];
        const float mean = sum / (float)depth;
        float vs = 0.0f;
        for (int z = 0; z < depth; ++z) {
            const float d = fabsf(xr[z] - mean);
            vs += d * d;
        }
        const float var = vs / (float)depth;
        const float rs = 1.0f / sqrtf(var + eps);
        for (int z = 0; z < depth; ++z) {
            const float inv = rs * (gamma ? gamma[z] : 1.0f);
            yr[z] = xr[z] * inv + ((beta ? beta[z] : 0.0f) - mean * inv);
        }
    }
}

/*
 * BatchNormalization with stored statistics along the last axis.
 * include/fdeep/layers/batch_normalization_layer.hpp:18-64, tensor.hpp:773-793.
 */
void fdo_batchnorm(const float* x, size_t positions, int c, const float* mean, const float* var,
    const float* gamma, const float* beta, float eps, float* y)
{
    for (size_t p = 0; p < positions; ++p)
        for (int z = 0; z < c; ++z) {
            const float inv = (1.0f / sqrtf(var[z] + eps)) * (gamma ? gamma[z] : 1.0f);
            y[p * c + z] = x[p * c + z] * inv + ((beta ? beta[z] : 0.0f) - mean[z] * inv);
        }
}

/* ReLU family, include/fdeep/layers/relu_layer.hpp:32-48 */
void fdo_relu(const float* x, size_t n, float max_value, float negative_slope, float threshold,
    float* y)
{
    if (negative_slope == 0.0f && threshold == 0.0f && max_value == FLT_MAX) {
        for (size_t i = 0; i < n; ++i)
            y[i] = x[i] > 0.0f ? x[i] : 0.0f;
        return;
    }
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        if (v >= max_value)
            y[i] = max_value;
        else if (threshold <= v && v < max_value)
            y[i] = v;
        else
            y[i] = negative_slope * (v - threshold);
    }
}

/* exact GELU, include/fdeep/recurrent_ops.hpp:73-76 */
void fdo_gelu(const float* x, size_t n, float* y)
{
    for (size_t i = 0; i < n; ++i)
        y[i] = 0.5f * x[i] * (1.0f + erff(x[i] / sqrtf(2.0f)));
}

/*
 * The other element-wise activations, one name each as the reference dispatches them
 * (include/fdeep/import_model.hpp:1649-1700); formulas from include/fdeep/recurrent_ops.hpp:24-86 and
 * include/fdeep/layers/<name>_layer.hpp.  p0 / p1 are the layer's parameters where it has any:
 * elu / celu alpha, leaky_relu slope, hard_shrink / soft_shrink threshold, squareplus b,
 * threshold (threshold, default value).  Returns -1 for a name the reference does not know.
 */
int fdo_activation(const char* name, float p0, float p1, const float* x, size_t n, float* y)
{
#define FDO_MAP(expr)                  \
    do {                               \
        for (size_t i = 0; i < n; ++i) { \
            const float v = x[i];      \
            y[i] = (expr);             \
        }                              \
        return 0;                      \
    } while (0)
    if (!strcmp(name, "tanh")) FDO_MAP(tanhf(v));
    if (!strcmp(name, "sigmoid")) FDO_MAP(1 / (1 + expf(-v)));
    if (!strcmp(name, "swish") || !strcmp(name, "silu")) FDO_MAP(v / (1 + expf(-v)));
    if (!strcmp(name, "hard_sigmoid")) FDO_MAP(v < -3 ? 0.0f : (v > 3 ? 1.0f : v / 6.0f + 0.5f));
    if (!strcmp(name, "selu"))
        FDO_MAP(1.0507009873554804934193349852946f * (v >= 0 ? v : 1.6732632423543772848170429916717f * (expf(v) - 1)));
    if (!strcmp(name, "elu") || !strcmp(name, "celu")) FDO_MAP(v >= 0 ? v : p0 * (expf(v) - 1));
    if (!strcmp(name, "exponential")) FDO_MAP(expf(v));
    if (!strcmp(name, "softsign")) FDO_MAP(v / (fabsf(v) + 1.0f));
    if (!strcmp(name, "softplus")) {
        const float threshold = logf(FLT_EPSILON) + 2; /* layers/softplus_layer.hpp */
        FDO_MAP(v > -threshold ? v : (v < threshold ? expf(v) : log1pf(expf(v))));
    }
    if (!strcmp(name, "leaky_relu")) FDO_MAP(v > 0 ? v : p0 * v);
    if (!strcmp(name, "hard_shrink")) FDO_MAP(fabsf(v) > p0 ? v : 0.0f);
    if (!strcmp(name, "soft_shrink")) FDO_MAP(v > p0 ? v - p0 : (v < -p0 ? v + p0 : 0.0f));
    if (!strcmp(name, "sparse_plus")) FDO_MAP(v <= -1 ? 0.0f : (v < 1 ? 0.25f * (v + 1.0f) * (v + 1.0f) : v));
    if (!strcmp(name, "squareplus")) FDO_MAP((v + sqrtf(v * v + p0)) / 2.0f);
    if (!strcmp(name, "tanh_shrink")) FDO_MAP(v - tanhf(v));
    if (!strcmp(name, "threshold")) FDO_MAP(v > p0 ? v : p1);
    if (!strcmp(name, "log_sigmoid")) FDO_MAP(logf(1 / (1 + expf(-v))));
    if (!strcmp(name, "hard_tanh")) FDO_MAP(v < -1 ? -1.0f : (v > 1 ? 1.0f : v));
    if (!strcmp(name, "log")) FDO_MAP(logf(v)); /* second half of log_softmax = log(softmax(x)) */
#undef FDO_MAP
    return -1;
}

/* element-wise merges of equal-shaped tensors: mult / subtract (include/fdeep/tensor.hpp:667-675),
 * max_tensors / min_tensors (:893-929); op 1 mul, 2 sub, 3 max, 4 min */
void fdo_combine(int op, const float* a, const float* b, size_t n, float* y)
{
    for (size_t i = 0; i < n; ++i)
        y[i] = op == 1 ? a[i] * b[i] : op == 2 ? a[i] - b[i] : op == 3 ? (a[i] > b[i] ? a[i] : b[i]) : (a[i] < b[i] ? a[i] : b[i]);
}

/* PReLU on a (h, w, c) sample: x > 0 ? x : alpha[pos] * x with alpha laid out over the axes that are not shared
 * (include/fdeep/layers/prelu_layer.hpp:46-66) */
void fdo_prelu(const float* x, int h, int w, int c, const float* alpha, int h_shared, int w_shared, int c_shared, float* y)
{
    const int aw = w_shared ? 1 : w, ac = c_shared ? 1 : c;
    for (int yy = 0; yy < h; ++yy)
        for (int xx = 0; xx < w; ++xx)
            for (int z = 0; z < c; ++z) {
                const size_t i = ((size_t)yy * w + xx) * c + z;
                const size_t pos = (size_t)(h_shared ? 0 : yy) * aw * ac + (size_t)(w_shared ? 0 : xx) * ac + (c_shared ? 0 : z);
                y[i] = x[i] > 0 ? x[i] : alpha[pos] * x[i];
            }
}

/*
 * Max / average 2-D pooling with TF padding; padded taps carry the lowest()
 * sentinel: ignored by max and left out of the average's divisor.
 * include/fdeep/layers/pooling_3d_layer.hpp:44-79, max_pooling_3d_layer.hpp:17-38,
 * average_pooling_3d_layer.hpp:17-42.  mode 0 = max, 1 = average.
 */
int fdo_pool2d(const float* in, int h, int w, int c, int ph, int pw, int sy, int sx,
    int pad_type, int mode, float* out, int* out_hw)
{
    int g[6];
    if (fdo_window_geometry(h, w, ph, pw, sy, sx, pad_type, g) != 0)
        return -1;
    out_hw[0] = g[4];
    out_hw[1] = g[5];
    if (!out)
        return 0;
    const float invalid = -FLT_MAX;
    for (int y = 0; y < g[4]; ++y)
        for (int x = 0; x < g[5]; ++x)
            for (int z = 0; z < c; ++z) {
                float val = mode == 0 ? -FLT_MAX : 0.0f;
                size_t divisor = 0;
                for (int yf = 0; yf < ph; ++yf) {
                    const int iy = sy * y + yf - g[0];
                    for (int xf = 0; xf < pw; ++xf) {
                        const int ix = sx * x + xf - g[2];
                        const float cur = (iy < 0 || iy >= h || ix < 0 || ix >= w)
                            ? invalid
                            : in[((size_t)iy * w + ix) * c + z];
                        if (mode == 0) {
                            val = cur > val ? cur : val;
                        } else if (cur != invalid) {
                            val += cur;
                            divisor += 1;
                        }
                    }
                }
                out[((size_t)y * g[5] + x) * c + z] = mode == 0 ? val : val / (float)divisor;
            }
    return 0;
}

/* GlobalAveragePooling, include/fdeep/layers/global_average_pooling_3d_layer.hpp:25-41;
 * GlobalMaxPooling, global_max_pooling_3d_layer.hpp (mode 0 = max, 1 = average). */
void fdo_global_pool(const float* in, size_t positions, int c, int mode, float* out)
{
    for (int z = 0; z < c; ++z) {
        float val = mode == 0 ? -FLT_MAX : 0.0f;
        for (size_t p = 0; p < positions; ++p) {
            const float cur = in[p * c + z];
            if (mode == 0)
                val = cur > val ? cur : val;
            else
                val += cur;
        }
        out[z] = mode == 0 ? val : val / (float)positions;
    }
}

/* element-wise sum of equal-shaped tensors, include/fdeep/tensor.hpp:642-680 */
void fdo_add(const float* a, const float* b, size_t n, float* y)
{
    for (size_t i = 0; i < n; ++i)
        y[i] = a[i] + b[i];
}

/* Embedding gather; ids are floats truncated to size_t, out of range is an error.
 * include/fdeep/layers/embedding_layer.hpp:38-58 */
int fdo_embedding(const float* ids, int count, const float* table, int input_dim, int output_dim,
    float* out)
{
    for (int i = 0; i < count; ++i) {
        const size_t id = (size_t)ids[i];
        if (id >= (size_t)input_dim)
            return -1;
        memcpy(out + (size_t)i * output_dim, table + id * output_dim, sizeof(float) * output_dim);
    }
    return 0;
}

/* first maximum wins, include/fdeep/tensor.hpp:281-302 */
size_t fdo_argmax(const float* x, size_t n)
{
    size_t best = 0;
    float bv = -FLT_MAX;
    for (size_t i = 0; i < n; ++i)
        if (x[i] > bv) {
            bv = x[i];
            best = i;
        }
    return best;
}

/*
 * MultiHeadAttention.  For every head h: per-head Dense on query / value / key
 * (slices along the H axis of the (D,H,dim) kernels), scores = Q * K^T,
 * scores *= 1/sqrt(key_dim), softmax over keys, times V; heads concatenated on
 * depth in head order; output Dense with kernel (H*dv, Dout).  No mask.
 * include/fdeep/layers/multi_head_attention_layer.hpp:34-110,
 * include/fdeep/tensor.hpp:814-884 (dot_product_tensors), 1165-1192 (softmax).
 * Weights in Keras order/shape: qw (D,H,dk) qb (H,dk) kw (D,H,dk) kb (H,dk)
 * vw (D,H,dv) vb (H,dv) ow (H,dv,Dout) ob (Dout); biases may be NULL.
 */
int fdo_mha(const float* query, int t, const float* value, const float* key, int s, int d,
    int heads, int dk, int dv, int dout,
    const float* qw, const float* qb, const float* kw, const float* kb,
    const float* vw, const float* vb, const float* ow, const float* ob, float* out)
{
    float* q = (float*)malloc(sizeof(float) * (size_t)t * dk);
    float* k = (float*)malloc(sizeof(float) * (size_t)s * dk);
    float* v = (float*)malloc(sizeof(float) * (size_t)s * dv);
    float* sc = (float*)malloc(sizeof(float) * (size_t)t * s);
    float* merged = (float*)malloc(sizeof(float) * (size_t)t * heads * dv);
    float* wh = (float*)malloc(sizeof(float) * (size_t)d * (dk > dv ? dk : dv));
    if (!q || !k || !v || !sc || !merged || !wh) {
        free(q); free(k); free(v); free(sc); free(merged); free(wh);
        return -2;
    }
    /* 1 / std::sqrt(size_t) is a double; the float score is multiplied in double and
     * narrowed on store (multi_head_attention_layer.hpp:92-93) */
    const double scale = 1.0 / sqrt((double)dk);
    for (int h = 0; h < heads; ++h) {
        /* per-head weight slice along H: W[:, h, :] */
        for (int i = 0; i < d; ++i)
            memcpy(wh + (size_t)i * dk, qw + ((size_t)i * heads + h) * dk, sizeof(float) * dk);
        fdo_dense(query, t, d, wh, qb ? qb + (size_t)h * dk : NULL, dk, q);
        for (int i = 0; i < d; ++i)
            memcpy(wh + (size_t)i * dv, vw + ((size_t)i * heads + h) * dv, sizeof(float) * dv);
        fdo_dense(value, s, d, wh, vb ? vb + (size_t)h * dv : NULL, dv, v);
        for (int i = 0; i < d; ++i)
            memcpy(wh + (size_t)i * dk, kw + ((size_t)i * heads + h) * dk, sizeof(float) * dk);
        fdo_dense(key, s, d, wh, kb ? kb + (size_t)h * dk : NULL, dk, k);
        for (int i = 0; i < t; ++i)
            for (int j = 0; j < s; ++j) {
                float acc = 0.0f;
                for (int z = 0; z < dk; ++z)
                    acc += q[(size_t)i * dk + z] * k[(size_t)j * dk + z];
                sc[(size_t)i * s + j] = (float)((double)acc * scale);
            }
        fdo_softmax(sc, t, s, sc);
        for (int i = 0; i < t; ++i) {
            float* o = merged + ((size_t)i * heads + h) * dv;
            for (int z = 0; z < dv; ++z)
                o[z] = 0.0f;
            for (int j = 0; j < s; ++j) {
                const float p = sc[(size_t)i * s + j];
                for (int z = 0; z < dv; ++z)
                    o[z] += p * v[(size_t)j * dv + z];
            }
        }
    }
    fdo_dense(merged, t, heads * dv, ow, ob, dout, out);
    free(q); free(k); free(v); free(sc); free(merged); free(wh);
    return 0;
}

/*
 * UpSampling2D by integer factors (layers/upsampling_2d_layer.hpp; resize2d_nearest / resize2d_bilinear,
 * include/fdeep/tensor.hpp:959-974, 997-1035).  Source coordinate of output row y: (y + 0.5) / scale - 0.5 with
 * scale = out / in in float.  Nearest rounds it to the closest index; for an integer factor f that coordinate lies
 * strictly inside (q - 0.5, q + 0.5) for y = q f + r, so every round-to-nearest rule (the reference calls
 * FunctionalPlus' round) gives q = y / f.  Bilinear clamps the coordinate to [0, extent], takes floor and floor + 1
 * (the latter clamped to the last index) and blends with weights formed as in the reference: the upper / left weight
 * in float, its complement and the products in double.
 */
void fdo_upsample2d(const float* in, int h, int w, int c, int fy, int fx, int bilinear, float* out)
{
    const int oh = h * fy, ow = w * fx;
    const float scale_y = (float)oh / (float)h, scale_x = (float)ow / (float)w;
    for (int y = 0; y < oh; ++y)
        for (int x = 0; x < ow; ++x)
            for (int z = 0; z < c; ++z) {
                float* dst = out + ((size_t)y * ow + x) * c + z;
                if (!bilinear) {
                    *dst = in[((size_t)(y / fy) * w + (x / fx)) * c + z];
                    continue;
                }
                float yi = ((float)y + 0.5f) / scale_y - 0.5f, xi = ((float)x + 0.5f) / scale_x - 0.5f;
                yi = yi < 0 ? 0 : yi;
                xi = xi < 0 ? 0 : xi;
                yi = yi > (float)h ? (float)h : yi;
                xi = xi > (float)w ? (float)w : xi;
                const int yt = (int)floorf(yi), xl = (int)floorf(xi);
                const int yb = yt + 1 < h - 1 ? yt + 1 : h - 1, xr = xl + 1 < w - 1 ? xl + 1 : w - 1;
                const int ytc = yt < h - 1 ? yt : h - 1, xlc = xl < w - 1 ? xl : w - 1; /* the coordinate stays below the extent, so this clamp never acts; it only guards the read */
                const float ft = (float)yb - yi, fl = (float)xr - xi;
                const double fb = 1.0 - ft, fr = 1.0 - fl;
                *dst = (float)(ft * fl * in[((size_t)ytc * w + xlc) * c + z] + ft * fr * in[((size_t)ytc * w + xr) * c + z]
                    + fb * fl * in[((size_t)yb * w + xlc) * c + z] + fb * fr * in[((size_t)yb * w + xr) * c + z]);
            }
}

/*
 * GroupQueryAttention: Q projected to hq heads, K / V to hkv heads (kernels (D, heads, hd), biases
 * (heads, hd)); query head h reads key/value head h / (hq / hkv); scores scaled by 1/sqrt(hd) in
 * float, softmax as exp(s - max) / sum; optional sigmoid gate (a second projection of the query)
 * multiplied onto the attention output; output kernel (hq, hd, dout).
 * include/fdeep/layers/group_query_attention_layer.hpp:62-220.  Biases / gate may be NULL.
 */
int fdo_gqa(const float* query, int t, const float* value, const float* key, int s, int d, int hd, int hq, int hkv,
    const float* qw, const float* qb, const float* kw, const float* kb, const float* gw, const float* gb,
    const float* vw, const float* vb, const float* ow, const float* ob, int dout, float* out)
{
    if (hkv <= 0 || hq % hkv != 0)
        return -1;
    const int group = hq / hkv;
    float* q = (float*)malloc(sizeof(float) * (size_t)t * hq * hd);
    float* g = gw ? (float*)malloc(sizeof(float) * (size_t)t * hq * hd) : NULL;
    float* k = (float*)malloc(sizeof(float) * (size_t)s * hkv * hd);
    float* v = (float*)malloc(sizeof(float) * (size_t)s * hkv * hd);
    float* attn = (float*)malloc(sizeof(float) * (size_t)t * hq * hd);
    float* sc = (float*)malloc(sizeof(float) * (size_t)s);
#define FDO_PROJECT(dst, src, rows, heads, w, b)                                  \
    for (int r = 0; r < rows; ++r)                                                \
        for (int h = 0; h < heads; ++h)                                           \
            for (int c = 0; c < hd; ++c) {                                        \
                float acc = 0;                                                    \
                for (int i = 0; i < d; ++i)                                       \
                    acc += src[(size_t)r * d + i] * w[((size_t)i * heads + h) * hd + c]; \
                if (b)                                                            \
                    acc += b[h * hd + c];                                         \
                dst[((size_t)r * heads + h) * hd + c] = acc;                      \
            }
    FDO_PROJECT(q, query, t, hq, qw, qb)
    FDO_PROJECT(k, key, s, hkv, kw, kb)
    FDO_PROJECT(v, value, s, hkv, vw, vb)
    if (gw)
        FDO_PROJECT(g, query, t, hq, gw, gb)
#undef FDO_PROJECT
    const float inv_sqrt = 1.0f / sqrtf((float)hd);
    for (int h = 0; h < hq; ++h) {
        const int hk = h / group;
        for (int tq = 0; tq < t; ++tq) {
            float mx = -INFINITY;
            for (int tk = 0; tk < s; ++tk) {
                float a = 0;
                for (int c = 0; c < hd; ++c)
                    a += q[((size_t)tq * hq + h) * hd + c] * k[((size_t)tk * hkv + hk) * hd + c];
                a *= inv_sqrt;
                sc[tk] = a;
                if (a > mx)
                    mx = a;
            }
            float sum = 0;
            for (int tk = 0; tk < s; ++tk) {
                sc[tk] = expf(sc[tk] - mx);
                sum += sc[tk];
            }
            for (int tk = 0; tk < s; ++tk)
                sc[tk] /= sum;
            for (int c = 0; c < hd; ++c) {
                float a = 0;
                for (int tk = 0; tk < s; ++tk)
                    a += sc[tk] * v[((size_t)tk * hkv + hk) * hd + c];
                attn[((size_t)tq * hq + h) * hd + c] = a;
            }
        }
    }
    if (g)
        for (size_t i = 0; i < (size_t)t * hq * hd; ++i)
            attn[i] *= 1.0f / (1.0f + expf(-g[i]));
    for (int r = 0; r < t; ++r)
        for (int o = 0; o < dout; ++o) {
            float a = 0;
            for (int i = 0; i < hq * hd; ++i)
                a += attn[(size_t)r * hq * hd + i] * ow[(size_t)i * dout + o];
            if (ob)
                a += ob[o];
            out[(size_t)r * dout + o] = a;
        }
    free(q); free(g); free(k); free(v); free(attn); free(sc);
    return 0;
}

/* RMSNormalization over the last `depth` elements of each row: x / sqrt(mean(x^2) + eps) * scale
 * (include/fdeep/layers/rms_normalization_layer.hpp:37-69); scale may be NULL */
void fdo_rmsnorm(const float* x, size_t rows, int depth, const float* scale, float eps, float* y)
{
    for (size_t r = 0; r < rows; ++r) {
        const float* xr = x + r * (size_t)depth;
        float ss = 0;
        for (int i = 0; i < depth; ++i)
            ss += xr[i] * xr[i];
        const float inv = 1.0f / sqrtf(ss / (float)depth + eps);
        for (int i = 0; i < depth; ++i)
            y[r * (size_t)depth + i] = xr[i] * inv * (scale ? scale[i] : 1.0f);
    }
}

/*
 * EinsumDense restricted to one contraction of the form used by the reference's
 * tests: out[rhs] = sum over summed chars of in[lhs] * kernel[rhs_kernel] (+ bias
 * laid out in rhs-char order over the chars named by bias_axes).  The leading
 * batch char of lhs/rhs is already stripped by the caller.  Index arithmetic is
 * the generic per-character decode of
 * include/fdeep/layers/einsum_dense_layer.hpp:155-250.
 * n_chars <= 16; sizes[i] is the extent of char i; *_idx list the char ids of each
 * operand in storage order; bias_idx lists bias chars in *rhs order*.
 */
int fdo_einsum_dense(const float* in, const int* in_idx, int in_rank,
    const float* kernel, const int* k_idx, int k_rank,
    const float* bias, const int* bias_idx, int bias_rank,
    const int* out_idx, int out_rank, const int* sum_idx, int sum_rank,
    const int* sizes, int n_chars, float* out)
{
    if (n_chars > 16)
        return -1;
    size_t out_vol = 1, sum_vol = 1;
    for (int i = 0; i < out_rank; ++i)
        out_vol *= (size_t)sizes[out_idx[i]];
    for (int i = 0; i < sum_rank; ++i)
        sum_vol *= (size_t)sizes[sum_idx[i]];
    int pos[16];
    for (size_t o = 0; o < out_vol; ++o) {
        size_t rem = o;
        for (int i = out_rank - 1; i >= 0; --i) {
            pos[out_idx[i]] = (int)(rem % (size_t)sizes[out_idx[i]]);
            rem /= (size_t)sizes[out_idx[i]];
        }
        float acc = 0.0f;
        for (size_t sidx = 0; sidx < sum_vol; ++sidx) {
            size_t r2 = sidx;
            for (int i = sum_rank - 1; i >= 0; --i) {
                pos[sum_idx[i]] = (int)(r2 % (size_t)sizes[sum_idx[i]]);
                r2 /= (size_t)sizes[sum_idx[i]];
            }
            size_t io = 0, ko = 0;
            for (int i = 0; i < in_rank; ++i)
                io = io * (size_t)sizes[in_idx[i]] + (size_t)pos[in_idx[i]];
            for (int i = 0; i < k_rank; ++i)
                ko = ko * (size_t)sizes[k_idx[i]] + (size_t)pos[k_idx[i]];
            acc += in[io] * kernel[ko];
        }
        if (bias) {
            size_t bo = 0;
            for (int i = 0; i < bias_rank; ++i)
                bo = bo * (size_t)sizes[bias_idx[i]] + (size_t)pos[bias_idx[i]];
            acc += bias[bo];
        }
        out[o] = acc;
    }
    return 0;
}
