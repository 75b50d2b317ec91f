// Strided tensor kernels for the layer forms that are not a plain row-major pass: EinsumDense
// with an arbitrary equation, element-wise Add with size-1 broadcasting on any axis,
// Concatenate, and LayerNormalization over axes that are not the trailing ones.  They are
// index-decoding kernels (one output element, or one normalisation group, per lane / wave) and
// HBM-bound; the regular cases of the same layers take the contiguous kernels instead.
#include <algorithm>
#include <string>
#include <vector>

#include "common.hpp"
#include "einsum.hpp"

namespace fdx {

struct EinsumDesc {
    int n_out, n_sum;
    int64_t od[6], oi[6], ok[6], ob[6]; // per output char: extent, stride in input / kernel / bias
    int64_t sd[4], si[4], sk[4];        // per summed char: extent, stride in input / kernel
};

// out[rhs] = sum over summed chars of in[lhs] * kernel[...] (+ bias), one output element per lane;
// the summed characters advance like an odometer so the inner loop has no divisions.
// include/fdeep/layers/einsum_dense_layer.hpp:169-196, 223-250
__global__ void einsum_kernel(const float* __restrict__ in, const float* __restrict__ kernel, const float* __restrict__ bias,
    float* __restrict__ out, EinsumDesc d, size_t total, Act act)
{
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        size_t rem = o;
        int64_t bi = 0, bk = 0, bb = 0;
        for (int i = d.n_out - 1; i >= 0; --i) {
            const int64_t c = (int64_t)(rem % (size_t)d.od[i]);
            rem /= (size_t)d.od[i];
            bi += c * d.oi[i];
            bk += c * d.ok[i];
            bb += c * d.ob[i];
        }
        float acc = 0.f;
        int64_t c0 = 0, c1 = 0, c2 = 0, c3 = 0;
        const int64_t e0 = d.n_sum > 0 ? d.sd[0] : 1, e1 = d.n_sum > 1 ? d.sd[1] : 1, e2 = d.n_sum > 2 ? d.sd[2] : 1,
                      e3 = d.n_sum > 3 ? d.sd[3] : 1;
        for (c0 = 0; c0 < e0; ++c0)
            for (c1 = 0; c1 < e1; ++c1)
                for (c2 = 0; c2 < e2; ++c2) {
                    const int64_t pi = bi + c0 * d.si[0] + c1 * d.si[1] + c2 * d.si[2];
                    const int64_t pk = bk + c0 * d.sk[0] + c1 * d.sk[1] + c2 * d.sk[2];
                    for (c3 = 0; c3 < e3; ++c3)
                        acc += in[pi + c3 * d.si[3]] * kernel[pk + c3 * d.sk[3]];
                }
        if (bias)
            acc += bias[bb];
        out[o] = apply_act(acc, act);
    }
}

struct BcastDesc {
    int64_t dims[6], sa[6], sb[6]; // output extents (batch first), operand strides (0 = repeated)
};

// include/fdeep/tensor.hpp:642-660: every axis of the two operands is equal or 1; the size-1 side repeats
template <int OP>
__device__ __forceinline__ float combine(float x, float y)
{
    switch (OP) {
    case FDX_COMBINE_MUL: return x * y;
    case FDX_COMBINE_SUB: return x - y;
    case FDX_COMBINE_MAX: return fmaxf(x, y);
    case FDX_COMBINE_MIN: return fminf(x, y);
    case FDX_COMBINE_PRELU: return x > 0.0f ? x : y * x;
    default: return x + y;
    }
}

template <int OP>
__global__ void bcast_combine_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out,
    BcastDesc d, size_t total, float scale, Act act)
{
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        size_t rem = o;
        int64_t pa = 0, pb = 0;
#pragma unroll
        for (int i = 5; i >= 0; --i) {
            const int64_t c = (int64_t)(rem % (size_t)d.dims[i]);
            rem /= (size_t)d.dims[i];
            pa += c * d.sa[i];
            pb += c * d.sb[i];
        }
        out[o] = apply_act(scale * combine<OP>(a[pa], b[pb]), act);
    }
}

// rows of `cols` floats copied into a wider row-major destination (row pitch ld_out)
__global__ void copy_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int64_t rows, int64_t cols, int64_t ld_out)
{
    const size_t total = (size_t)rows * (size_t)cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / (size_t)cols, c = i % (size_t)cols;
        out[r * (size_t)ld_out + c] = in[i];
    }
}

struct NormDesc {
    int n_keep, n_norm;
    int64_t kd[6], ks[6]; // kept axes (batch first): extent, stride
    int64_t nd[5], ns[5]; // normalised axes in storage order: extent, stride
};

// One wave per group (= one position on the kept axes).  Mean, then the biased variance as the
// mean of squared differences, then x * inv + (beta - mean * inv) with inv = gamma / sqrt(var + eps)
// (include/fdeep/tensor.hpp:758-793, layers/layer_normalization_layer.hpp:37-61); gamma / beta are
// indexed by the position on the normalised axes.
// RMS: no mean, x / sqrt(mean(x^2) + eps) * gamma (include/fdeep/layers/rms_normalization_layer.hpp:37-69).
template <bool RMS>
__global__ __launch_bounds__(256) void layernorm_axes_kernel(const float* __restrict__ x, float* __restrict__ out, NormDesc d,
    int64_t groups, int64_t count, const float* __restrict__ gamma, const float* __restrict__ beta, float eps)
{
    const int lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= groups)
        return;
    int64_t base = 0;
    {
        int64_t rem = g;
        for (int i = d.n_keep - 1; i >= 0; --i) {
            base += (rem % d.kd[i]) * d.ks[i];
            rem /= d.kd[i];
        }
    }
    auto offset = [&](int64_t e) {
        int64_t off = base;
        for (int i = d.n_norm - 1; i >= 0; --i) {
            off += (e % d.nd[i]) * d.ns[i];
            e /= d.nd[i];
        }
        return off;
    };
    float s = 0.f;
    if (!RMS)
        for (int64_t e = lane; e < count; e += 64)
            s += x[offset(e)];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        s += __shfl_xor(s, o, 64);
    const float mean = RMS ? 0.f : s / (float)count;
    float v = 0.f;
    for (int64_t e = lane; e < count; e += 64) {
        const float df = x[offset(e)] - mean;
        v += df * df;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    const float rstd = 1.0f / sqrtf(v / (float)count + eps);
    for (int64_t e = lane; e < count; e += 64) {
        const int64_t off = offset(e);
        const float inv = (gamma ? gamma[e] : 1.0f) * rstd;
        out[off] = x[off] * inv + ((beta ? beta[e] : 0.0f) - mean * inv);
    }
}

struct PermuteDesc {
    int64_t od[6], is[6]; // output extents (batch first) and, per output axis, the stride of its source axis
};

// permute_tensor (include/fdeep/tensor.hpp:526-549): output axis i is input axis dims[i] - 1
__global__ void permute_kernel(const float* __restrict__ in, float* __restrict__ out, PermuteDesc d, size_t total)
{
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        size_t rem = o;
        int64_t pi = 0;
#pragma unroll
        for (int i = 5; i >= 0; --i) {
            pi += (int64_t)(rem % (size_t)d.od[i]) * d.is[i];
            rem /= (size_t)d.od[i];
        }
        out[o] = in[pi];
    }
}

// crop_tensor (include/fdeep/tensor.hpp:586-610) on [n][h][w][c]
__global__ void crop2d_kernel(const float* __restrict__ in, float* __restrict__ out, int h, int w, int c, int top, int left,
    int oh, int ow, size_t total)
{
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        const int z = (int)(o % (size_t)c);
        size_t rest = o / (size_t)c;
        const int x = (int)(rest % (size_t)ow);
        rest /= (size_t)ow;
        const int y = (int)(rest % (size_t)oh);
        const size_t img = rest / (size_t)oh;
        out[o] = in[((img * h + (y + top)) * (size_t)w + (x + left)) * c + z];
    }
}

// dilate_tensor (include/fdeep/tensor.hpp:612-640) on [n][h][w][c]: input pixel (y, x) lands on (y*ry + oy, x*rx + ox), every
// other output pixel is zero; one thread per output element, so the zeros are written by the same pass
__global__ void dilate2d_kernel(const float* __restrict__ in, float* __restrict__ out, int h, int w, int c, int ry, int rx, int oy,
    int ox, int oh, int ow, size_t total)
{
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        const int z = (int)(o % (size_t)c);
        size_t rest = o / (size_t)c;
        const int x = (int)(rest % (size_t)ow) - ox;
        rest /= (size_t)ow;
        const int y = (int)(rest % (size_t)oh) - oy;
        const size_t img = rest / (size_t)oh;
        float v = 0.f;
        if (y >= 0 && x >= 0 && y % ry == 0 && x % rx == 0 && y / ry < h && x / rx < w)
            v = in[((img * h + (size_t)(y / ry)) * w + (size_t)(x / rx)) * c + z];
        out[o] = v;
    }
}

// resize2d_nearest / resize2d_bilinear for integer factors (include/fdeep/tensor.hpp:959-974, 997-1035): source
// coordinate (y + 0.5) / factor - 0.5; nearest rounds it (= y / factor for integer factors), bilinear clamps it to
// [0, extent] and blends the four neighbours, the lower / right one clamped to the last row / column
template <bool BILINEAR>
__global__ void resize2d_kernel(const float* __restrict__ in, float* __restrict__ out, int h, int w, int c, int fy, int fx,
    size_t total)
{
    const int oh = h * fy, ow = w * fx;
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        const int z = (int)(o % (size_t)c);
        size_t rest = o / (size_t)c;
        const int x = (int)(rest % (size_t)ow);
        rest /= (size_t)ow;
        const int y = (int)(rest % (size_t)oh);
        const float* img = in + (rest / (size_t)oh) * (size_t)h * w * c;
        if (!BILINEAR) {
            out[o] = img[((size_t)(y / fy) * w + (x / fx)) * c + z];
        } else {
            float yi = ((float)y + 0.5f) / (float)fy - 0.5f, xi = ((float)x + 0.5f) / (float)fx - 0.5f;
            yi = fminf(fmaxf(yi, 0.f), (float)h);
            xi = fminf(fmaxf(xi, 0.f), (float)w);
            const int yt = (int)floorf(yi), xl = (int)floorf(xi);
            const int yb = min(h - 1, yt + 1), xr = min(w - 1, xl + 1);
            const int ytc = min(yt, h - 1), xlc = min(xl, w - 1);
            const double ft = (double)((float)yb - yi), fb = 1.0 - ft, fl = (double)((float)xr - xi), fr = 1.0 - fl;
            const double v = ft * fl * img[((size_t)ytc * w + xlc) * c + z] + ft * fr * img[((size_t)ytc * w + xr) * c + z]
                + fb * fl * img[((size_t)yb * w + xlc) * c + z] + fb * fr * img[((size_t)yb * w + xr) * c + z];
            out[o] = (float)v;
        }
    }
}

static int grid_of(size_t work_items, int block)
{
    size_t g = (work_items + block - 1) / block;
    const size_t cap = 256 * 16;
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

// Shared by the C entry point and the model executor.  in_dims: extents of the trailing lhs
// characters (the batch is simply the first of them); the kernel keeps the layout of the file.
fdx_status einsum_launch(EinsumSpec& spec, const float* in, const float* kernel, const float* bias, const Act& act, float* out)
{
    EinsumDesc d {};
    d.n_out = (int)spec.rhs.size();
    d.n_sum = (int)spec.summed.size();
    for (int i = 0; i < d.n_out; ++i) {
        const char c = spec.rhs[(size_t)i];
        d.od[i] = spec.size.at(c);
        d.oi[i] = spec.stride_in(spec.lhs, c);
        d.ok[i] = spec.stride_in(spec.ker, c);
        d.ob[i] = spec.stride_in(spec.bias_chars, c);
    }
    for (int i = 0; i < 4; ++i) {
        d.sd[i] = 1;
        d.si[i] = d.sk[i] = 0;
    }
    // the longest summed axis goes innermost only by position: keep the equation's order
    for (int i = 0; i < d.n_sum; ++i) {
        const char c = spec.summed[(size_t)i];
        const int slot = 4 - d.n_sum + i; // right-aligned so the innermost loop is the last summed char
        d.sd[slot] = spec.size.at(c);
        d.si[slot] = spec.stride_in(spec.lhs, c);
        d.sk[slot] = spec.stride_in(spec.ker, c);
    }
    d.n_sum = 4;
    const int64_t total = spec.volume_of(spec.rhs), sum_vol = spec.volume_of(spec.summed);
    FDX_REQUIRE(total > 0 && sum_vol > 0, "einsum_dense: empty operand");
    profile_begin();
    hipLaunchKernelGGL(einsum_kernel, dim3(grid_of((size_t)total, 256)), dim3(256), 0, stream(), in, kernel,
        spec.bias_chars.empty() ? nullptr : bias, out, d, (size_t)total, act);
    profile_end("einsum_dense_f32", 2.0 * (double)total * (double)sum_vol,
        4.0 * ((double)spec.volume_of(spec.lhs) + (double)spec.volume_of(spec.ker) + (double)total));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

} // namespace fdx

using namespace fdx;

extern "C" fdx_status fdx_einsum_dense_f32(const char* equation, const char* bias_axes, const float* in, int in_rank,
    const int64_t* in_dims, const float* kernel, int kernel_rank, const int64_t* kernel_dims, const float* bias,
    const int64_t* full_output_shape, const fdx_act* act, float* out, int* out_rank, int64_t* out_dims)
{
    FDX_REQUIRE(equation && in && in_dims && kernel && kernel_dims && out, "einsum_dense: null argument");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(in_rank >= 1 && in_rank <= 6 && kernel_rank >= 1 && kernel_rank <= 6, "einsum_dense: ranks must be 1..6");
    EinsumSpec spec;
    std::string err;
    if (!spec.parse(equation, bias_axes ? bias_axes : "", err)) {
        set_error("%s", err.c_str());
        return FDX_ERR_INVALID;
    }
    std::vector<int64_t> full;
    if (full_output_shape)
        full.assign(full_output_shape, full_output_shape + spec.rhs.size());
    if (!spec.derive_sizes(std::vector<int64_t>(kernel_dims, kernel_dims + kernel_rank),
            std::vector<int64_t>(in_dims, in_dims + in_rank), full, err)) {
        set_error("%s", err.c_str());
        return FDX_ERR_INVALID;
    }
    FDX_REQUIRE(spec.bias_chars.empty() || bias, "einsum_dense: bias_axes given without a bias");
    if (out_rank)
        *out_rank = (int)spec.rhs.size();
    if (out_dims)
        for (size_t i = 0; i < spec.rhs.size(); ++i)
            out_dims[i] = spec.size.at(spec.rhs[i]);
    return einsum_launch(spec, in, kernel, bias, make_act(act), out);
}

extern "C" fdx_status fdx_broadcast_add_f32(const float* a, const int64_t* a_dims5, const float* b, const int64_t* b_dims5,
    int batch, const fdx_act* act, float* out, int64_t* out_dims5)
{
    return fdx_broadcast_combine_f32(FDX_COMBINE_ADD, a, a_dims5, b, b_dims5, 0, batch, 1.0f, act, out, out_dims5);
}

extern "C" fdx_status fdx_broadcast_combine_f32(int op, const float* a, const int64_t* a_dims5, const float* b,
    const int64_t* b_dims5, int b_shared, int batch, float scale, const fdx_act* act, float* out, int64_t* out_dims5)
{
    FDX_REQUIRE(a && b && a_dims5 && b_dims5 && out && batch > 0, "broadcast_combine: bad arguments");
    FDX_REQUIRE(op >= FDX_COMBINE_ADD && op <= FDX_COMBINE_PRELU, "broadcast_combine: unknown operation %d", op);
    FDX_REQUIRE_EPILOGUE_ACT(act);
    BcastDesc d {};
    int64_t va = 1, vb = 1, vo = 1;
    for (int i = 0; i < 5; ++i) {
        const int64_t x = a_dims5[i], y = b_dims5[i];
        FDX_REQUIRE(x > 0 && y > 0 && (x == y || x == 1 || y == 1), "Invalid shapes for combining tensors.");
        d.dims[i + 1] = std::max(x, y);
        va *= x;
        vb *= y;
        vo *= d.dims[i + 1];
        if (out_dims5)
            out_dims5[i] = d.dims[i + 1];
    }
    int64_t sa = 1, sb = 1;
    for (int i = 4; i >= 0; --i) {
        d.sa[i + 1] = a_dims5[i] == 1 ? 0 : sa;
        d.sb[i + 1] = b_dims5[i] == 1 ? 0 : sb;
        sa *= a_dims5[i];
        sb *= b_dims5[i];
    }
    d.dims[0] = batch;
    d.sa[0] = va;
    d.sb[0] = b_shared ? 0 : vb;
    const size_t total = (size_t)batch * (size_t)vo;
    const Act ac = make_act(act);
    const dim3 grid(grid_of(total, 256)), block(256);
    profile_begin();
    switch (op) {
    case FDX_COMBINE_MUL: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_MUL>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    case FDX_COMBINE_SUB: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_SUB>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    case FDX_COMBINE_MAX: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_MAX>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    case FDX_COMBINE_MIN: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_MIN>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    case FDX_COMBINE_PRELU: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_PRELU>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    default: hipLaunchKernelGGL(bcast_combine_kernel<FDX_COMBINE_ADD>, grid, block, 0, stream(), a, b, out, d, total, scale, ac); break;
    }
    profile_end("broadcast_combine_f32", 0.0, 4.0 * ((double)batch * va + (double)(b_shared ? 1 : batch) * vb + (double)total));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_concat_f32(const float* const* ins, int n_inputs, const int64_t* inner, int64_t outer, float* out)
{
    FDX_REQUIRE(ins && inner && out && n_inputs > 0 && outer > 0, "concat: bad arguments");
    int64_t ld = 0;
    for (int i = 0; i < n_inputs; ++i) {
        FDX_REQUIRE(ins[i] && inner[i] > 0, "concat: bad input %d", i);
        ld += inner[i];
    }
    int64_t off = 0;
    for (int i = 0; i < n_inputs; ++i) {
        const size_t total = (size_t)outer * (size_t)inner[i];
        profile_begin();
        hipLaunchKernelGGL(copy_rows_kernel, dim3(grid_of(total, 256)), dim3(256), 0, stream(), ins[i], out + off, outer, inner[i], ld);
        profile_end("concat_f32", 0.0, 8.0 * (double)total);
        FDX_LAUNCH_CHECK();
        off += inner[i];
    }
    return FDX_OK;
}

static fdx_status norm_axes(const float* x, int batch, const int64_t* dims5, unsigned axes_mask, const float* gamma,
    const float* beta, float eps, float* out, bool rms)
{
    FDX_REQUIRE(x && dims5 && out && batch > 0 && axes_mask != 0 && axes_mask < 32, "layernorm_axes: bad arguments");
    int64_t vol = 1;
    for (int i = 0; i < 5; ++i) {
        FDX_REQUIRE(dims5[i] > 0, "layernorm_axes: bad extent");
        vol *= dims5[i];
    }
    // trailing axes (ignoring size-1 axes around them) are one contiguous row: the fast kernel
    {
        int64_t depth = 1;
        int i = 4;
        for (; i >= 0 && ((axes_mask >> i) & 1u || dims5[i] == 1); --i)
            if ((axes_mask >> i) & 1u)
                depth *= dims5[i];
        bool rest_kept = true;
        for (int j = i; j >= 0; --j)
            if (((axes_mask >> j) & 1u) && dims5[j] != 1)
                rest_kept = false;
        if (!rms && rest_kept && depth < (1LL << 31))
            return fdx_layernorm_f32(x, (int64_t)batch * vol / depth, (int)depth, gamma, beta, eps, out);
    }
    NormDesc d {};
    d.kd[0] = batch;
    d.ks[0] = vol;
    d.n_keep = 1;
    int64_t stride = vol, count = 1, groups = batch;
    for (int i = 0; i < 5; ++i) {
        stride /= dims5[i];
        if ((axes_mask >> i) & 1u) {
            d.nd[d.n_norm] = dims5[i];
            d.ns[d.n_norm++] = stride;
            count *= dims5[i];
        } else {
            d.kd[d.n_keep] = dims5[i];
            d.ks[d.n_keep++] = stride;
            groups *= dims5[i];
        }
    }
    profile_begin();
    if (rms)
        hipLaunchKernelGGL(layernorm_axes_kernel<true>, dim3((unsigned)((groups + 3) / 4)), dim3(256), 0, stream(), x, out, d, groups,
            count, gamma, nullptr, eps);
    else
        hipLaunchKernelGGL(layernorm_axes_kernel<false>, dim3((unsigned)((groups + 3) / 4)), dim3(256), 0, stream(), x, out, d, groups,
            count, gamma, beta, eps);
    profile_end(rms ? "rmsnorm_axes_f32" : "layernorm_axes_f32", 0.0, 8.0 * (double)batch * (double)vol);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_layernorm_axes_f32(const float* x, int batch, const int64_t* dims5, unsigned axes_mask, const float* gamma,
    const float* beta, float eps, float* out)
{
    return norm_axes(x, batch, dims5, axes_mask, gamma, beta, eps, out, false);
}

extern "C" fdx_status fdx_rmsnorm_axes_f32(const float* x, int batch, const int64_t* dims5, unsigned axes_mask, const float* scale,
    float eps, float* out)
{
    return norm_axes(x, batch, dims5, axes_mask, scale, nullptr, eps, out, true);
}

extern "C" fdx_status fdx_permute_f32(const float* in, int batch, int rank, const int64_t* dims, const int* perm, float* out)
{
    FDX_REQUIRE(in && dims && perm && out && batch > 0 && rank >= 1 && rank <= 5, "permute: bad arguments");
    int64_t istride[5], vol = 1;
    bool seen[5] = { false, false, false, false, false };
    for (int i = rank - 1; i >= 0; --i) {
        FDX_REQUIRE(dims[i] > 0, "permute: bad extent");
        istride[i] = vol;
        vol *= dims[i];
    }
    PermuteDesc d {};
    for (int i = 0; i < 6; ++i) {
        d.od[i] = 1;
        d.is[i] = 0;
    }
    d.od[0] = batch;
    d.is[0] = vol;
    for (int i = 0; i < rank; ++i) {
        FDX_REQUIRE(perm[i] >= 0 && perm[i] < rank && !seen[perm[i]], "Invalid dims for permute.");
        seen[perm[i]] = true;
        d.od[6 - rank + i] = dims[perm[i]];
        d.is[6 - rank + i] = istride[perm[i]];
    }
    const size_t total = (size_t)batch * (size_t)vol;
    profile_begin();
    hipLaunchKernelGGL(permute_kernel, dim3(grid_of(total, 256)), dim3(256), 0, stream(), in, out, d, total);
    profile_end("permute_f32", 0.0, 8.0 * (double)total);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_crop2d_nhwc_f32(const float* in, int n, int h, int w, int c, int top, int bottom, int left, int right,
    float* out)
{
    FDX_REQUIRE(in && out && n > 0 && h > 0 && w > 0 && c > 0 && top >= 0 && bottom >= 0 && left >= 0 && right >= 0
            && top + bottom < h && left + right < w,
        "crop2d: bad arguments");
    const int oh = h - top - bottom, ow = w - left - right;
    const size_t total = (size_t)n * oh * ow * c;
    profile_begin();
    hipLaunchKernelGGL(crop2d_kernel, dim3(grid_of(total, 256)), dim3(256), 0, stream(), in, out, h, w, c, top, left, oh, ow, total);
    profile_end("crop2d_f32", 0.0, 8.0 * (double)total);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_dilate2d_nhwc_f32(const float* in, int n, int h, int w, int c, int rate_y, int rate_x, int trailing_zeros,
    float* out)
{
    FDX_REQUIRE(in && out && n > 0 && h > 0 && w > 0 && c > 0 && rate_y > 0 && rate_x > 0, "dilate2d: bad arguments");
    const bool unit = rate_y == 1 && rate_x == 1; // the reference returns the input itself for rate (1, 1)
    const int ey = (trailing_zeros && !unit) ? rate_y - 1 : 0, ex = (trailing_zeros && !unit) ? rate_x - 1 : 0;
    const int oh = (h - 1) * rate_y + 1 + ey, ow = (w - 1) * rate_x + 1 + ex;
    const size_t total = (size_t)n * oh * ow * c;
    profile_begin();
    hipLaunchKernelGGL(dilate2d_kernel, dim3(grid_of(total, 256)), dim3(256), 0, stream(), in, out, h, w, c, rate_y, rate_x,
        ey - ey / 2, ex - ex / 2, oh, ow, total);
    profile_end("dilate2d_f32", 0.0, 4.0 * ((double)total + (double)n * h * w * c));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_upsample2d_nhwc_f32(const float* in, int n, int h, int w, int c, int factor_y, int factor_x, int bilinear,
    float* out)
{
    FDX_REQUIRE(in && out && n > 0 && h > 0 && w > 0 && c > 0 && factor_y > 0 && factor_x > 0, "upsample2d: bad arguments");
    const size_t total = (size_t)n * h * factor_y * w * factor_x * c;
    profile_begin();
    if (bilinear)
        hipLaunchKernelGGL(resize2d_kernel<true>, dim3(grid_of(total, 256)), dim3(256), 0, stream(), in, out, h, w, c, factor_y,
            factor_x, total);
    else
        hipLaunchKernelGGL(resize2d_kernel<false>, dim3(grid_of(total, 256)), dim3(256), 0, stream(), in, out, h, w, c, factor_y,
            factor_x, total);
    profile_end("upsample2d_f32", 0.0, 4.0 * ((double)total + (double)n * h * w * c));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
