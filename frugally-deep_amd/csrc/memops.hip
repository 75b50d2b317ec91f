// Memory-bound forward kernels (gfx950): depthwise conv, pooling, element-wise glue,
// LayerNorm, softmax, embedding gather, argmax, transpose.  All are channel-innermost
// (NHWC) so consecutive lanes touch consecutive addresses; rows are reduced with wave64
// shuffles and, across waves, a small LDS exchange.
#include <algorithm>
#include <cfloat>
#include <cstdlib>
#include <mutex>
#include <vector>
#include "common.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// block-wide reductions for blocks of up to 1024 threads; every thread gets the result
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* smem)
{
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (nw == 1)
        return v;
    __syncthreads();
    if (lane == 0)
        smem[wave] = v;
    __syncthreads();
    float r = smem[0];
    for (int i = 1; i < nw; ++i)
        r = IS_MAX ? fmaxf(r, smem[i]) : r + smem[i];
    return r;
}

// ------------------------------------------------------------------ depthwise conv
// One thread per (pixel, VEC channels): VEC = 4 uses 16-byte loads on activations and on
// the [kh][kw][c] filter.
template <int VEC>
__global__ void dwconv_kernel(const float* __restrict__ in, const float* __restrict__ wts,
    const float* __restrict__ bias, float* __restrict__ out, int n, int h, int w, int c, int kh, int kw,
    int sy, int sx, int dy, int dx, int pad_top, int pad_left, int oh, int ow, Act act)
{
    const int cv = c / VEC;
    const int64_t total = (int64_t)n * oh * ow * cv;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int cq = (int)(idx % cv);
        int64_t pix = idx / cv;
        const int ox = (int)(pix % ow);
        pix /= ow;
        const int oy = (int)(pix % oh);
        const int img = (int)(pix / oh);
        const int c0 = cq * VEC;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v)
            acc[v] = bias ? bias[c0 + v] : 0.f;
        const float* ib = in + (int64_t)img * h * w * c;
        for (int fy = 0; fy < kh; ++fy) {
            const int iy = oy * sy - pad_top + fy * dy;
            if (iy < 0 || iy >= h)
                continue;
            for (int fx = 0; fx < kw; ++fx) {
                const int ix = ox * sx - pad_left + fx * dx;
                if (ix < 0 || ix >= w)
                    continue;
                const float* ip = ib + ((int64_t)iy * w + ix) * c + c0;
                const float* wp = wts + ((int64_t)fy * kw + fx) * c + c0;
                if (VEC == 4) {
                    const f32x4 a = *reinterpret_cast<const f32x4*>(ip);
                    const f32x4 b = *reinterpret_cast<const f32x4*>(wp);
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        acc[v] += a[v] * b[v];
                } else {
                    acc[0] += ip[0] * wp[0];
                }
            }
        }
        float* op = out + (((int64_t)img * oh + oy) * ow + ox) * c + c0;
        if (VEC == 4) {
            float r[4] = { acc[0], acc[1], acc[2], acc[3] };
            apply_act_block(r, act);
            *reinterpret_cast<f32x4*>(op) = f32x4 { r[0], r[1], r[2], r[3] };
        } else {
            op[0] = apply_act(acc[0], act);
        }
    }
}


// 3x3, dilation 1, four channels per lane and TX consecutive output columns per thread: the nine
// filter vectors stay in registers and each input row segment is loaded once for all TX outputs
// (the plain kernel above issues 18 loads per output vector, which caps it well below HBM speed).
template <int STRIDE, int TX>
__global__ __launch_bounds__(256) void dwconv3x3_kernel(const float* __restrict__ in, const float* __restrict__ wts,
    const float* __restrict__ bias, float* __restrict__ out, int n, int h, int w, int c, int pad_top, int pad_left,
    int oh, int ow, Act act)
{
    constexpr int COLS = (TX - 1) * STRIDE + 3;
    const unsigned cv = (unsigned)c / 4, xt = (unsigned)(ow + TX - 1) / TX;
    // item index in 32 bits (the host launches this kernel only below 2^31 items): a 64-bit division costs several
    // times the arithmetic of an item
    const unsigned total = (unsigned)n * (unsigned)oh * xt * cv;
    for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        unsigned rest = idx / cv;
        const int cq = (int)(idx - rest * cv);
        unsigned rest2 = rest / xt;
        const int ox0 = (int)(rest - rest2 * xt) * TX;
        const int img = (int)(rest2 / (unsigned)oh);
        const int oy = (int)(rest2 - (unsigned)img * (unsigned)oh);
        const int c0 = cq * 4;
        f32x4 wv[9];
#pragma unroll
        for (int t = 0; t < 9; ++t)
            wv[t] = *reinterpret_cast<const f32x4*>(wts + (int64_t)t * c + c0);
        f32x4 acc[TX];
        const f32x4 b4 = bias ? *reinterpret_cast<const f32x4*>(bias + c0) : f32x4 { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
        for (int j = 0; j < TX; ++j)
            acc[j] = b4;
        const float* ib = in + (int64_t)img * h * w * c + c0;
        const int ix0 = ox0 * STRIDE - pad_left;
#pragma unroll
        for (int fy = 0; fy < 3; ++fy) {
            const int iy = oy * STRIDE - pad_top + fy;
            if (iy < 0 || iy >= h)
                continue;
            const float* row = ib + (int64_t)iy * w * c;
            f32x4 col[COLS];
#pragma unroll
            for (int k = 0; k < COLS; ++k) {
                const int ix = ix0 + k;
                col[k] = (ix >= 0 && ix < w) ? *reinterpret_cast<const f32x4*>(row + (int64_t)ix * c) : f32x4 { 0.f, 0.f, 0.f, 0.f };
            }
#pragma unroll
            for (int j = 0; j < TX; ++j)
#pragma unroll
                for (int fx = 0; fx < 3; ++fx)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        acc[j][v] += col[j * STRIDE + fx][v] * wv[fy * 3 + fx][v];
        }
        float* op = out + (((int64_t)img * oh + oy) * ow + ox0) * c + c0;
        float r[TX * 4];
#pragma unroll
        for (int j = 0; j < TX; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                r[j * 4 + v] = acc[j][v];
        apply_act_block(r, act);
#pragma unroll
        for (int j = 0; j < TX; ++j)
            if (ox0 + j < ow)
                *reinterpret_cast<f32x4*>(op + (int64_t)j * c) = f32x4 { r[j * 4], r[j * 4 + 1], r[j * 4 + 2], r[j * 4 + 3] };
    }
}

// The same 3x3 stride-1 stencil with a window that slides down the image: a lane owns TX output columns of four
// channels and walks RY output rows, keeping three input rows in registers, so every input value is loaded once per
// column tile (plus its two frame columns) instead of once per output row that touches it -- 1.3 to 1.7 loads per
// output where the row-at-a-time kernel above issues 3.75.  Meant for the small feature maps (14 x 14, 7 x 7) with
// many channels, where that kernel's three-fold row reuse has to come from the caches; it needs enough (image, row
// tile, column tile, channel quad) items to fill the chip, which the launcher checks.
template <int TX, int RY>
__global__ __launch_bounds__(256) void dwconv3x3_slide_kernel(const float* __restrict__ in, const float* __restrict__ wts,
    const float* __restrict__ bias, float* __restrict__ out, int n, int h, int w, int c, int pad_top, int pad_left,
    int oh, int ow, Act act)
{
    constexpr int COLS = TX + 2;
    const unsigned cv = (unsigned)c / 4, xt = (unsigned)(ow + TX - 1) / TX, yt = (unsigned)(oh + RY - 1) / RY;
    const unsigned total = (unsigned)n * yt * xt * cv;
    for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        unsigned rest = idx / cv;
        const int cq = (int)(idx - rest * cv);
        unsigned rest2 = rest / xt;
        const int ox0 = (int)(rest - rest2 * xt) * TX;
        const int img = (int)(rest2 / yt);
        const int oy0 = (int)(rest2 - (unsigned)img * yt) * RY;
        const int c0 = cq * 4;
        f32x4 wv[9];
#pragma unroll
        for (int t = 0; t < 9; ++t)
            wv[t] = *reinterpret_cast<const f32x4*>(wts + (int64_t)t * c + c0);
        const f32x4 b4 = bias ? *reinterpret_cast<const f32x4*>(bias + c0) : f32x4 { 0.f, 0.f, 0.f, 0.f };
        const float* ib = in + (int64_t)img * h * w * c + c0;
        const int ix0 = ox0 - pad_left;
        auto load_row = [&](f32x4 (&dst)[COLS], int iy) {
            const bool row_ok = iy >= 0 && iy < h;
            const float* row = ib + (int64_t)(row_ok ? iy : 0) * w * c;
#pragma unroll
            for (int k = 0; k < COLS; ++k) {
                const int ix = ix0 + k;
                dst[k] = (row_ok && ix >= 0 && ix < w) ? *reinterpret_cast<const f32x4*>(row + (int64_t)ix * c) : f32x4 { 0.f, 0.f, 0.f, 0.f };
            }
        };
        f32x4 win[3][COLS]; // input rows iy, iy + 1, iy + 2 of the current output row, in slots (r, r + 1, r + 2) % 3
        load_row(win[0], oy0 - pad_top);
        load_row(win[1], oy0 - pad_top + 1);
#pragma unroll
        for (int r = 0; r < RY; ++r) {
            load_row(win[(r + 2) % 3], oy0 - pad_top + r + 2);
            const int oy = oy0 + r;
            f32x4 acc[TX];
#pragma unroll
            for (int j = 0; j < TX; ++j)
                acc[j] = b4;
#pragma unroll
            for (int fy = 0; fy < 3; ++fy)
#pragma unroll
                for (int j = 0; j < TX; ++j)
#pragma unroll
                    for (int fx = 0; fx < 3; ++fx)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            acc[j][v] += win[(r + fy) % 3][j + fx][v] * wv[fy * 3 + fx][v];
            float res[TX * 4];
#pragma unroll
            for (int j = 0; j < TX; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    res[j * 4 + v] = acc[j][v];
            apply_act_block(res, act);
            if (oy < oh) {
                float* op = out + (((int64_t)img * oh + oy) * ow + ox0) * c + c0;
#pragma unroll
                for (int j = 0; j < TX; ++j)
                    if (ox0 + j < ow)
                        *reinterpret_cast<f32x4*>(op + (int64_t)j * c) = f32x4 { res[j * 4], res[j * 4 + 1], res[j * 4 + 2], res[j * 4 + 3] };
            }
        }
    }
}

// ------------------------------------------------------------------ pooling
// One lane per (output pixel, VEC channels); VEC = 4 moves 16 bytes per access.
template <int VEC>
__global__ void pool2d_kernel(const float* __restrict__ in, float* __restrict__ out, int n, int h, int w, int c,
    int ph, int pw, int sy, int sx, int pad_top, int pad_left, int zt, int zl, int zb, int zr, int oh, int ow, int mode)
{
    const int cv = c / VEC;
    const int64_t total = (int64_t)n * oh * ow * cv;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int ch = (int)(idx % cv) * VEC;
        int64_t pix = idx / cv;
        const int ox = (int)(pix % ow);
        pix /= ow;
        const int oy = (int)(pix % oh);
        const int img = (int)(pix / oh);
        float val[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v)
            val[v] = mode == 0 ? -FLT_MAX : 0.f;
        int div = 0;
        for (int fy = 0; fy < ph; ++fy) {
            const int iy = oy * sy + fy - pad_top;
            for (int fx = 0; fx < pw; ++fx) {
                const int ix = ox * sx + fx - pad_left;
                float cur[VEC];
                if (iy >= 0 && iy < h && ix >= 0 && ix < w) {
                    const float* src = in + (((int64_t)img * h + iy) * w + ix) * c + ch;
                    if (VEC == 4) {
                        const f32x4 t = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
                        for (int v = 0; v < VEC; ++v)
                            cur[v] = t[v];
                    } else
                        cur[0] = src[0];
                } else if (iy >= -zt && iy < h + zb && ix >= -zl && ix < w + zr) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v)
                        cur[v] = 0.f; // inside a folded explicit zero-padding frame: a real zero
                } else
                    continue; // TF padding: ignored by max, excluded from the average
#pragma unroll
                for (int v = 0; v < VEC; ++v)
                    val[v] = mode == 0 ? fmaxf(val[v], cur[v]) : val[v] + cur[v];
                ++div;
            }
        }
        float* dst = out + (((int64_t)img * oh + oy) * ow + ox) * c + ch;
        if (VEC == 4) {
            f32x4 r;
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                r[v] = mode == 0 ? val[v] : val[v] / (float)div;
            *reinterpret_cast<f32x4*>(dst) = r;
        } else
            dst[0] = mode == 0 ? val[0] : val[0] / (float)div;
    }
}

// one workgroup per (sample, 64-channel group); 4 waves stride over positions
__global__ __launch_bounds__(256) void global_pool_kernel(const float* __restrict__ in, float* __restrict__ out,
    int positions, int c, int mode)
{
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cgroups = (c + 63) / 64;
    const int img = blockIdx.x / cgroups, ch = (blockIdx.x % cgroups) * 64 + lane;
    float val = mode == 0 ? -FLT_MAX : 0.f;
    if (ch < c) {
        const float* p = in + (int64_t)img * positions * c + ch;
        for (int i = wave; i < positions; i += 4) {
            const float cur = p[(int64_t)i * c];
            val = mode == 0 ? fmaxf(val, cur) : val + cur;
        }
    }
    part[wave][lane] = val;
    __syncthreads();
    if (wave == 0 && ch < c) {
        // positions are summed in four interleaved partial sums, then combined
        float r = part[0][lane];
        for (int i = 1; i < 4; ++i)
            r = mode == 0 ? fmaxf(r, part[i][lane]) : r + part[i][lane];
        out[(int64_t)img * c + ch] = mode == 0 ? r : r / (float)positions;
    }
}

// ------------------------------------------------------------------ element-wise
template <int VEC>
__global__ void add_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out,
    size_t count, size_t b_count, Act act)
{
    const size_t nv = count / VEC;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < nv; i += (size_t)gridDim.x * blockDim.x) {
        if (VEC == 4) {
            const f32x4 x = reinterpret_cast<const f32x4*>(a)[i];
            const f32x4 y = reinterpret_cast<const f32x4*>(b)[b_count == count ? i : i % (b_count / 4)];
            float r[4] = { x[0] + y[0], x[1] + y[1], x[2] + y[2], x[3] + y[3] };
            apply_act_block(r, act);
            reinterpret_cast<f32x4*>(out)[i] = f32x4 { r[0], r[1], r[2], r[3] };
        } else {
            out[i] = apply_act(a[i] + b[b_count == count ? i : i % b_count], act);
        }
    }
}

template <int VEC>
__global__ void act_kernel(const float* __restrict__ x, float* __restrict__ out, size_t count, Act act)
{
    const size_t nv = count / VEC;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < nv; i += (size_t)gridDim.x * blockDim.x) {
        if (VEC == 4) {
            const f32x4 v = reinterpret_cast<const f32x4*>(x)[i];
            f32x4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                r[e] = apply_act_full(v[e], act);
            reinterpret_cast<f32x4*>(out)[i] = r;
        } else {
            out[i] = apply_act_full(x[i], act);
        }
    }
}

__global__ void affine_kernel(const float* __restrict__ x, float* __restrict__ out, size_t count, int c,
    const float* __restrict__ scale, const float* __restrict__ shift, Act act)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        const int ch = (int)(i % (size_t)c);
        out[i] = apply_act(x[i] * scale[ch] + shift[ch], act);
    }
}

__global__ void zero_pad_kernel(const float* __restrict__ in, float* __restrict__ out, int n, int h, int w, int c,
    int pt, int pl, int oh, int ow)
{
    const int64_t total = (int64_t)n * oh * ow * c;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int ch = (int)(idx % c);
        int64_t pix = idx / c;
        const int ox = (int)(pix % ow);
        pix /= ow;
        const int oy = (int)(pix % oh);
        const int img = (int)(pix / oh);
        const int iy = oy - pt, ix = ox - pl;
        out[idx] = (iy >= 0 && iy < h && ix >= 0 && ix < w) ? in[(((int64_t)img * h + iy) * w + ix) * c + ch] : 0.f;
    }
}

// in: rows x cols with row stride ld_in; out: cols x rows packed.  blockIdx.z walks independent matrices.
__global__ void transpose_kernel(const float* __restrict__ in, float* __restrict__ out, int rows, int cols,
    int64_t ld_in, int64_t in_batch, int64_t out_batch)
{
    __shared__ float tile[32][33];
    in += (int64_t)blockIdx.z * in_batch;
    out += (int64_t)blockIdx.z * out_batch;
    const int bx = blockIdx.x * 32, by = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 256 threads: 8 rows per pass
    for (int r = ty; r < 32; r += 8)
        if (by + r < rows && bx + tx < cols)
            tile[r][tx] = in[(int64_t)(by + r) * ld_in + bx + tx];
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (bx + r < cols && by + tx < rows)
            out[(int64_t)(bx + r) * rows + by + tx] = tile[tx][r];
}

// out[r][:] = in[offset + r * row_stride + :]  (last position of every sequence, for instance)
__global__ void gather_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int depth, int64_t row_stride,
    int64_t offset)
{
    const float* src = in + offset + (int64_t)blockIdx.x * row_stride;
    float* dst = out + (int64_t)blockIdx.x * depth;
    for (int z = threadIdx.x; z < depth; z += blockDim.x)
        dst[z] = src[z];
}

// ------------------------------------------------------------------ LayerNorm
// One wave per row when depth <= 64*MAXV (row held in registers: read once, write once);
// the generic kernel re-reads the row for larger depths.
template <int MAXV>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(const float* __restrict__ x, float* __restrict__ out,
    int64_t rows, int depth, const float* __restrict__ gamma, const float* __restrict__ beta, float eps)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4LL + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const float* xr = x + row * depth;
    float v[MAXV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int z = lane + i * 64;
        v[i] = z < depth ? xr[z] : 0.f;
        s += v[i];
    }
    const float mean = wave_sum(s) / (float)depth;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int z = lane + i * 64;
        const float d = z < depth ? v[i] - mean : 0.f;
        q += d * d;
    }
    const float rs = 1.0f / sqrtf(wave_sum(q) / (float)depth + eps);
    float* orow = out + row * depth;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int z = lane + i * 64;
        if (z < depth) {
            const float inv = rs * (gamma ? gamma[z] : 1.f);
            orow[z] = v[i] * inv + ((beta ? beta[z] : 0.f) - mean * inv);
        }
    }
}

// Same, 16 bytes per lane and access (depth a multiple of 4, at most 256 * NV): a row is NV wave-wide loads.
template <int NV>
__global__ __launch_bounds__(256) void layernorm_wave4_kernel(const float* __restrict__ x, float* __restrict__ out,
    int64_t rows, int depth, const float* __restrict__ gamma, const float* __restrict__ beta, float eps)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = blockIdx.x * 4LL + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const float* xr = x + row * depth;
    f32x4 v[NV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int z = (lane + i * 64) * 4;
        v[i] = z < depth ? *reinterpret_cast<const f32x4*>(xr + z) : f32x4 { 0.f, 0.f, 0.f, 0.f };
        s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
    }
    const float mean = wave_sum(s) / (float)depth;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
        if ((lane + i * 64) * 4 < depth)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float d = v[i][e] - mean;
                q += d * d;
            }
    const float rs = 1.0f / sqrtf(wave_sum(q) / (float)depth + eps);
    float* orow = out + row * depth;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int z = (lane + i * 64) * 4;
        if (z < depth) {
            const f32x4 g = gamma ? *reinterpret_cast<const f32x4*>(gamma + z) : f32x4 { 1.f, 1.f, 1.f, 1.f };
            const f32x4 b = beta ? *reinterpret_cast<const f32x4*>(beta + z) : f32x4 { 0.f, 0.f, 0.f, 0.f };
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float inv = rs * g[e];
                o[e] = v[i][e] * inv + (b[e] - mean * inv);
            }
            *reinterpret_cast<f32x4*>(orow + z) = o;
        }
    }
}

__global__ __launch_bounds__(256) void layernorm_block_kernel(const float* __restrict__ x, float* __restrict__ out,
    int depth, const float* __restrict__ gamma, const float* __restrict__ beta, float eps)
{
    __shared__ float smem[16];
    const float* xr = x + (int64_t)blockIdx.x * depth;
    float s = 0.f;
    for (int z = threadIdx.x; z < depth; z += blockDim.x)
        s += xr[z];
    const float mean = block_reduce<false>(s, smem) / (float)depth;
    float q = 0.f;
    for (int z = threadIdx.x; z < depth; z += blockDim.x) {
        const float d = xr[z] - mean;
        q += d * d;
    }
    const float rs = 1.0f / sqrtf(block_reduce<false>(q, smem) / (float)depth + eps);
    float* orow = out + (int64_t)blockIdx.x * depth;
    for (int z = threadIdx.x; z < depth; z += blockDim.x) {
        const float inv = rs * (gamma ? gamma[z] : 1.f);
        orow[z] = xr[z] * inv + ((beta ? beta[z] : 0.f) - mean * inv);
    }
}

// ------------------------------------------------------------------ softmax
// exp(x - m - log(sum exp(x - m))) with infinities mapped to 0, the reference's form.
// THREADS = 64: four rows per 256-thread workgroup, one wave each; THREADS = 256: one row
// per workgroup.  `visible` limits a row to its first entries (causal prefix); the rest is 0.
template <int THREADS>
__global__ __launch_bounds__(256) void softmax_kernel(const float* __restrict__ x, float* __restrict__ out,
    int64_t rows, int depth, int causal_period, int causal_offset)
{
    __shared__ float smem[16];
    const int tid = THREADS == 64 ? (threadIdx.x & 63) : threadIdx.x;
    const int64_t row = THREADS == 64 ? blockIdx.x * 4LL + (threadIdx.x >> 6) : blockIdx.x;
    if (row >= rows)
        return;
    int visible = depth;
    if (causal_period > 0) {
        visible = (int)(row % causal_period) + 1 + causal_offset;
        visible = visible > depth ? depth : visible;
    }
    const float* xr = x + row * depth;
    float* orow = out + row * depth;
    float m = -FLT_MAX;
    for (int z = tid; z < visible; z += THREADS)
        m = fmaxf(m, xr[z]);
    m = THREADS == 64 ? wave_max(m) : block_reduce<true>(m, smem);
    float s = 0.f;
    for (int z = tid; z < visible; z += THREADS)
        s += expf(xr[z] - m);
    s = THREADS == 64 ? wave_sum(s) : block_reduce<false>(s, smem);
    const float ls = logf(s);
    for (int z = tid; z < depth; z += THREADS) {
        float r = 0.f;
        if (z < visible) {
            r = expf(xr[z] - m - ls);
            r = isinf(r) ? 0.f : r;
        }
        orow[z] = r;
    }
}

// ------------------------------------------------------------------ embedding / argmax
__global__ void embedding_kernel(const float* __restrict__ ids, const float* __restrict__ table,
    float* __restrict__ out, int64_t count, int input_dim, int output_dim, int* __restrict__ err)
{
    const int64_t row = blockIdx.x;
    if (row >= count)
        return;
    const float f = ids[row];
    // float -> size_t truncation; negative or too large ids are out of range
    int64_t id = (f >= 0.f && f < 9.0e18f) ? (int64_t)f : -1;
    const bool ok = id >= 0 && id < input_dim;
    if (!ok && err && threadIdx.x == 0)
        atomicExch(err, 1);
    const float* src = table + (ok ? id : 0) * (int64_t)output_dim;
    float* dst = out + row * (int64_t)output_dim;
    for (int z = threadIdx.x; z < output_dim; z += blockDim.x)
        dst[z] = ok ? src[z] : 0.f;
}

// out[row] = embed_a[ids_a[row]] + embed_b[ids_b[row]] is left to the add kernel; kept simple.

__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ x, int64_t rows, int depth,
    int32_t* __restrict__ out_idx, float* __restrict__ out_val, float* __restrict__ out_idx_f)
{
    __shared__ float sv[4];
    __shared__ int si[4];
    const float* xr = x + (int64_t)blockIdx.x * depth;
    float best = -FLT_MAX;
    int bi = 0x7fffffff;
    for (int z = threadIdx.x; z < depth; z += blockDim.x) {
        const float v = xr[z];
        if (v > best) { // strict: the first maximum wins within this thread's ascending walk
            best = v;
            bi = z;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > best || (ov == best && oi < bi)) {
            best = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        sv[wave] = best;
        si[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < (int)(blockDim.x >> 6); ++i)
            if (sv[i] > best || (sv[i] == best && si[i] < bi)) {
                best = sv[i];
                bi = si[i];
            }
        if (bi == 0x7fffffff)
            bi = 0; // all entries are -FLT_MAX or NaN: the reference's initial position
        if (out_idx)
            out_idx[blockIdx.x] = bi;
        if (out_val)
            out_val[blockIdx.x] = best;
        if (out_idx_f)
            out_idx_f[blockIdx.x] = (float)bi;
    }
}

static int grid_for(size_t work_items, int block)
{
    size_t g = (work_items + block - 1) / block;
    const size_t cap = 256 * 16; // 16 workgroups per CU keep HBM busy; grid-stride covers the rest
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

} // namespace fdx

using namespace fdx;

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" fdx_status fdx_dwconv2d_nhwc_f32(const float* in, int n, int h, int w, int c,
    const float* weights_hwc, const float* bias, int kh, int kw,
    int sy, int sx, int dy, int dx, int pad_top, int pad_left, int out_h, int out_w,
    const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && weights_hwc && out, "dwconv2d: null pointer");
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0 && sy > 0 && sx > 0 && dy > 0 && dx > 0
            && out_h > 0 && out_w > 0 && pad_top >= 0 && pad_left >= 0,
        "dwconv2d: bad shape");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    const Act a = make_act(act);
    const bool vec = c % 4 == 0 && al16(in) && al16(weights_hwc) && al16(out);
    const size_t items = (size_t)n * out_h * out_w * (vec ? c / 4 : c);
    profile_begin();
    const bool k3 = vec && kh == 3 && kw == 3 && dy == 1 && dx == 1 && sy == sx && (sy == 1 || sy == 2) && (!bias || al16(bias))
        && (uint64_t)n * out_h * ((out_w + 3) / 4) * (c / 4) < (1ull << 31); // 32-bit item index in the 3x3 kernel
    // the sliding-window form wherever its (image, row tile, column tile, channel quad) items fill the chip; tiles of 7
    // where they divide the extent and 8 does not (14 x 14, 7 x 7), row tiles of 4 where taller ones leave too few items
    static const bool slide_on = [] { const char* e = std::getenv("FDX_DW_SLIDE"); return !(e && e[0] == '0'); }();
    const int tx_s = out_w % 7 == 0 && out_w % 8 != 0 ? 7 : 8;
    int ry_s = out_h % 7 == 0 && out_h % 8 != 0 ? 7 : 8;
    auto slide_items_for = [&](int ry) { return (size_t)n * ((out_h + ry - 1) / ry) * ((out_w + tx_s - 1) / tx_s) * (c / 4); };
    if (slide_items_for(ry_s) < 256 * 256)
        ry_s = 4;
    const size_t slide_items = slide_items_for(ry_s);
    const bool slide = k3 && sy == 1 && slide_on && slide_items >= 256 * 16;
#define FDX_DW_SLIDE_LAUNCH(TX_, RY_)                                                                                                  \
    hipLaunchKernelGGL((dwconv3x3_slide_kernel<TX_, RY_>), dim3(grid_for(slide_items, 256)), dim3(256), 0, stream(), in, weights_hwc, bias, out, \
        n, h, w, c, pad_top, pad_left, out_h, out_w, a)
    if (slide && tx_s == 7 && ry_s == 7)
        FDX_DW_SLIDE_LAUNCH(7, 7);
    else if (slide && tx_s == 8 && ry_s == 8)
        FDX_DW_SLIDE_LAUNCH(8, 8);
    else if (slide && tx_s == 7 && ry_s == 8)
        FDX_DW_SLIDE_LAUNCH(7, 8);
    else if (slide && tx_s == 8 && ry_s == 7)
        FDX_DW_SLIDE_LAUNCH(8, 7);
    else if (slide && tx_s == 7)
        FDX_DW_SLIDE_LAUNCH(7, 4);
    else if (slide)
        FDX_DW_SLIDE_LAUNCH(8, 4);
#undef FDX_DW_SLIDE_LAUNCH
    else if (k3 && sy == 1)
        hipLaunchKernelGGL((dwconv3x3_kernel<1, 8>), dim3(grid_for((size_t)n * out_h * ((out_w + 7) / 8) * (c / 4), 256)), dim3(256), 0,
            stream(), in, weights_hwc, bias, out, n, h, w, c, pad_top, pad_left, out_h, out_w, a);
    else if (k3)
        hipLaunchKernelGGL((dwconv3x3_kernel<2, 4>), dim3(grid_for((size_t)n * out_h * ((out_w + 3) / 4) * (c / 4), 256)), dim3(256), 0,
            stream(), in, weights_hwc, bias, out, n, h, w, c, pad_top, pad_left, out_h, out_w, a);
    else if (vec)
        hipLaunchKernelGGL(dwconv_kernel<4>, dim3(grid_for(items, 256)), dim3(256), 0, stream(), in, weights_hwc, bias,
            out, n, h, w, c, kh, kw, sy, sx, dy, dx, pad_top, pad_left, out_h, out_w, a);
    else
        hipLaunchKernelGGL(dwconv_kernel<1>, dim3(grid_for(items, 256)), dim3(256), 0, stream(), in, weights_hwc, bias,
            out, n, h, w, c, kh, kw, sy, sx, dy, dx, pad_top, pad_left, out_h, out_w, a);
    profile_end("dwconv_f32", 0.0, 4.0 * ((double)n * h * w * c + (double)n * out_h * out_w * c + (double)kh * kw * c));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_pool2d_nhwc_f32(const float* in, int n, int h, int w, int c, int ph, int pw, int sy, int sx,
    int pad_top, int pad_left, int zero_top, int zero_left, int zero_bottom, int zero_right,
    int out_h, int out_w, int mode, float* out)
{
    FDX_REQUIRE(in && out, "pool2d: null pointer");
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && ph > 0 && pw > 0 && sy > 0 && sx > 0 && out_h > 0 && out_w > 0,
        "pool2d: bad shape");
    FDX_REQUIRE(mode == 0 || mode == 1, "pool2d: mode must be 0 (max) or 1 (average)");
    const size_t items = (size_t)n * out_h * out_w * c;
    profile_begin();
    if (c % 4 == 0 && al16(in) && al16(out))
        hipLaunchKernelGGL(pool2d_kernel<4>, dim3(grid_for(items / 4, 256)), dim3(256), 0, stream(), in, out, n, h, w, c, ph, pw,
            sy, sx, pad_top, pad_left, zero_top, zero_left, zero_bottom, zero_right, out_h, out_w, mode);
    else
        hipLaunchKernelGGL(pool2d_kernel<1>, dim3(grid_for(items, 256)), dim3(256), 0, stream(), in, out, n, h, w, c, ph, pw,
            sy, sx, pad_top, pad_left, zero_top, zero_left, zero_bottom, zero_right, out_h, out_w, mode);
    profile_end("pool2d_f32", 0.0, 4.0 * ((double)n * h * w * c + (double)items));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_global_pool_f32(const float* in, int n, int positions, int c, int mode, float* out)
{
    FDX_REQUIRE(in && out && n > 0 && positions > 0 && c > 0, "global_pool: bad arguments");
    FDX_REQUIRE(mode == 0 || mode == 1, "global_pool: mode must be 0 (max) or 1 (average)");
    profile_begin();
    hipLaunchKernelGGL(global_pool_kernel, dim3(n * ((c + 63) / 64)), dim3(256), 0, stream(), in, out, positions, c, mode);
    profile_end("global_pool_f32", 0.0, 4.0 * ((double)n * positions * c + (double)n * c));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_eltwise_add_f32(const float* a, const float* b, size_t count, size_t b_count,
    const fdx_act* act, float* out)
{
    FDX_REQUIRE(a && b && out && count > 0 && b_count > 0 && count % b_count == 0, "eltwise_add: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    const Act ac = make_act(act);
    const bool vec = count % 4 == 0 && b_count % 4 == 0 && al16(a) && al16(b) && al16(out);
    profile_begin();
    if (vec)
        hipLaunchKernelGGL(add_kernel<4>, dim3(grid_for(count / 4, 256)), dim3(256), 0, stream(), a, b, out, count, b_count, ac);
    else
        hipLaunchKernelGGL(add_kernel<1>, dim3(grid_for(count, 256)), dim3(256), 0, stream(), a, b, out, count, b_count, ac);
    profile_end("eltwise_add_f32", 0.0, 4.0 * (2.0 * count + b_count));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_activation_f32(const float* x, size_t count, const fdx_act* act, float* out)
{
    FDX_REQUIRE(x && out && count > 0, "activation: bad arguments");
    FDX_REQUIRE(!act || (act->kind >= 0 && act->kind < FDX_ACT_COUNT), "activation: unknown kind %d", act ? act->kind : 0);
    const Act ac = make_act(act);
    const bool vec = count % 4 == 0 && al16(x) && al16(out);
    profile_begin();
    if (vec)
        hipLaunchKernelGGL(act_kernel<4>, dim3(grid_for(count / 4, 256)), dim3(256), 0, stream(), x, out, count, ac);
    else
        hipLaunchKernelGGL(act_kernel<1>, dim3(grid_for(count, 256)), dim3(256), 0, stream(), x, out, count, ac);
    profile_end("activation_f32", 0.0, 8.0 * count);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_channel_affine_f32(const float* x, size_t positions, int c, const float* scale,
    const float* shift, const fdx_act* act, float* out)
{
    FDX_REQUIRE(x && out && scale && shift && positions > 0 && c > 0, "channel_affine: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    const size_t count = positions * (size_t)c;
    profile_begin();
    hipLaunchKernelGGL(affine_kernel, dim3(grid_for(count, 256)), dim3(256), 0, stream(), x, out, count, c, scale, shift,
        make_act(act));
    profile_end("channel_affine_f32", 0.0, 8.0 * count);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_zero_pad2d_nhwc_f32(const float* in, int n, int h, int w, int c, int pt, int pb, int pl, int pr,
    float* out)
{
    FDX_REQUIRE(in && out && n > 0 && h > 0 && w > 0 && c > 0 && pt >= 0 && pb >= 0 && pl >= 0 && pr >= 0,
        "zero_pad2d: bad arguments");
    const int oh = h + pt + pb, ow = w + pl + pr;
    const size_t items = (size_t)n * oh * ow * c;
    profile_begin();
    hipLaunchKernelGGL(zero_pad_kernel, dim3(grid_for(items, 256)), dim3(256), 0, stream(), in, out, n, h, w, c, pt, pl, oh, ow);
    profile_end("zero_pad_f32", 0.0, 4.0 * ((double)n * h * w * c + (double)items));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

namespace fdx {
fdx_status transpose_launch(const float* in, int batch, int rows, int cols, int64_t ld_in, int64_t in_batch, float* out)
{
    FDX_REQUIRE(in && out && rows > 0 && cols > 0 && batch > 0 && batch <= 65535 && ld_in >= cols, "transpose: bad arguments");
    hipLaunchKernelGGL(transpose_kernel, dim3((cols + 31) / 32, (rows + 31) / 32, batch), dim3(256), 0, stream(), in, out,
        rows, cols, ld_in, in_batch, (int64_t)rows * cols);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

__global__ void positions_kernel(float* __restrict__ out, int batch, int t, int start)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < batch * t)
        out[i] = (float)(start + i % t);
}

// out[b][j] = start + j : the position ids of `t` new tokens of every sequence
fdx_status positions_launch(float* out, int batch, int t, int start)
{
    FDX_REQUIRE(out && batch > 0 && t > 0 && start >= 0, "positions: bad arguments");
    hipLaunchKernelGGL(positions_kernel, dim3((batch * t + 255) / 256), dim3(256), 0, stream(), out, batch, t, start);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status gather_rows_launch(const float* in, int64_t rows, int depth, int64_t row_stride, int64_t offset, float* out)
{
    FDX_REQUIRE(in && out && rows > 0 && depth > 0, "gather_rows: bad arguments");
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)rows), dim3(256), 0, stream(), in, out, depth, row_stride, offset);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
}

extern "C" fdx_status fdx_transpose_f32(const float* in, int rows, int cols, float* out)
{
    return fdx::transpose_launch(in, 1, rows, cols, cols, 0, out);
}

extern "C" fdx_status fdx_layernorm_f32(const float* x, int64_t rows, int depth, const float* gamma, const float* beta,
    float eps, float* out)
{
    FDX_REQUIRE(x && out && rows > 0 && depth > 0, "layernorm: bad arguments");
    profile_begin();
    const dim3 g4((unsigned)((rows + 3) / 4));
    auto a16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    if (depth % 4 == 0 && depth <= 1024 && a16(x) && a16(out) && a16(gamma) && a16(beta)) {
        if (depth <= 256)
            hipLaunchKernelGGL(layernorm_wave4_kernel<1>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
        else if (depth <= 512)
            hipLaunchKernelGGL(layernorm_wave4_kernel<2>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
        else if (depth <= 768)
            hipLaunchKernelGGL(layernorm_wave4_kernel<3>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
        else
            hipLaunchKernelGGL(layernorm_wave4_kernel<4>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
    } else if (depth <= 256)
        hipLaunchKernelGGL(layernorm_wave_kernel<4>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
    else if (depth <= 1024)
        hipLaunchKernelGGL(layernorm_wave_kernel<16>, g4, dim3(256), 0, stream(), x, out, rows, depth, gamma, beta, eps);
    else
        hipLaunchKernelGGL(layernorm_block_kernel, dim3((unsigned)rows), dim3(256), 0, stream(), x, out, depth, gamma, beta, eps);
    profile_end("layernorm_f32", 0.0, 8.0 * rows * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_softmax_f32(const float* x, int64_t rows, int depth, int causal_period, int causal_offset,
    float* out)
{
    FDX_REQUIRE(x && out && rows > 0 && depth > 0 && causal_period >= 0 && causal_offset >= 0, "softmax: bad arguments");
    profile_begin();
    if (depth <= 1024)
        hipLaunchKernelGGL(softmax_kernel<64>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream(), x, out, rows, depth,
            causal_period, causal_offset);
    else
        hipLaunchKernelGGL(softmax_kernel<256>, dim3((unsigned)rows), dim3(256), 0, stream(), x, out, rows, depth,
            causal_period, causal_offset);
    profile_end("softmax_f32", 0.0, 8.0 * rows * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" fdx_status fdx_embedding_f32(const float* ids, int64_t count, const float* table, int input_dim, int output_dim,
    float* out, int* error_flag_dev)
{
    FDX_REQUIRE(ids && table && out && count > 0 && input_dim > 0 && output_dim > 0, "embedding: bad arguments");
    profile_begin();
    hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)count), dim3(output_dim >= 256 ? 256 : 64), 0, stream(), ids, table, out,
        count, input_dim, output_dim, error_flag_dev);
    profile_end("embedding_f32", 0.0, 8.0 * count * output_dim);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

namespace fdx {
fdx_status argmax_launch(const float* x, int64_t rows, int depth, int32_t* out_idx, float* out_val, float* out_idx_f)
{
    FDX_REQUIRE(x && rows > 0 && depth > 0, "argmax: bad arguments");
    profile_begin();
    hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)rows), dim3(256), 0, stream(), x, rows, depth, out_idx, out_val, out_idx_f);
    profile_end("argmax_f32", 0.0, 4.0 * rows * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
}

extern "C" fdx_status fdx_argmax_f32(const float* x, int64_t rows, int depth, int32_t* out_idx, float* out_val)
{
    return fdx::argmax_launch(x, rows, depth, out_idx, out_val, nullptr);
}

// ---- shader-clock probe (a measurement aid; nothing in the reference corresponds to it)
//
// One lane on a stream of its own records the shader cycle counter and the constant-rate wall counter once per
// period while the library stream runs its work; the ratio of their steps is the clock the compute units ran at
// during that period.  The wait between samples sleeps and is bounded, and the kernel ends after `samples` periods
// whatever else happens.
namespace fdx {
__global__ void clock_probe_kernel(long long* out, int samples, long long period_ticks)
{
    long long next = wall_clock64();
    for (int i = 0; i < samples; ++i) {
        out[2 * i] = clock64();
        out[2 * i + 1] = wall_clock64();
        next += period_ticks;
        for (int spin = 0; spin < (1 << 18) && wall_clock64() < next; ++spin)
            __builtin_amdgcn_s_sleep(16);
    }
}

static std::mutex g_probe_mutex;
static hipStream_t g_probe_stream = nullptr;
static long long* g_probe_buf = nullptr;
static int g_probe_samples = 0;
constexpr int kProbeMaxSamples = 1 << 16;
}

extern "C" fdx_status fdx_clock_probe_start(int samples, int period_us)
{
    FDX_REQUIRE(samples >= 2 && samples <= kProbeMaxSamples && period_us >= 10 && period_us <= 100000,
        "clock_probe_start: 2..65536 samples, period 10..100000 us");
    // the probe kernel ends only by itself, and fdx_clock_probe_stop waits for it: keep its whole run within ten seconds
    FDX_REQUIRE((long long)samples * period_us <= 10LL * 1000 * 1000,
        "clock_probe_start: samples x period is %lld us; a probe may run for at most 10 s", (long long)samples * period_us);
    (void)stream(); // the library is initialised on its device
    std::lock_guard<std::mutex> lock(g_probe_mutex);
    FDX_REQUIRE(g_probe_samples == 0, "clock_probe_start: a probe is already running; call fdx_clock_probe_stop first");
    if (!g_probe_stream)
        FDX_HIP(hipStreamCreateWithFlags(&g_probe_stream, hipStreamNonBlocking));
    if (!g_probe_buf)
        FDX_HIP(hipMalloc(&g_probe_buf, (size_t)kProbeMaxSamples * 2 * sizeof(long long)));
    int dev = 0, khz = 0;
    FDX_HIP(hipGetDevice(&dev));
    FDX_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    FDX_REQUIRE(khz > 0, "clock_probe_start: the device reports no wall clock rate");
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(1), 0, g_probe_stream, g_probe_buf, samples,
        (long long)khz * period_us / 1000);
    FDX_LAUNCH_CHECK();
    g_probe_samples = samples;
    return FDX_OK;
}

extern "C" fdx_status fdx_clock_probe_stop(double window_ms, double* mean_ghz, double* min_ghz, double* max_ghz)
{
    FDX_REQUIRE(mean_ghz && min_ghz && max_ghz && window_ms > 0, "clock_probe_stop: bad arguments");
    std::lock_guard<std::mutex> lock(g_probe_mutex);
    FDX_REQUIRE(g_probe_samples > 0, "clock_probe_stop: no probe was started");
    const int n = g_probe_samples;
    g_probe_samples = 0;
    FDX_HIP(hipStreamSynchronize(g_probe_stream));
    std::vector<long long> h((size_t)n * 2);
    FDX_HIP(hipMemcpy(h.data(), g_probe_buf, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    int dev = 0, khz = 0;
    FDX_HIP(hipGetDevice(&dev));
    FDX_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    const double window_ticks = window_ms * khz;
    double lo = 1e30, hi = 0.0;
    long long c_first = h[0], w_first = h[1], c_last = h[0], w_last = h[1];
    for (int i = 1; i < n; ++i) {
        const long long dw = h[2 * i + 1] - h[2 * i - 1], dc = h[2 * i] - h[2 * i - 2];
        if ((double)(h[2 * i + 1] - w_first) > window_ticks)
            break;
        if (dw <= 0)
            continue;
        const double ghz = (double)dc / (double)dw * khz * 1e-6;
        lo = std::min(lo, ghz);
        hi = std::max(hi, ghz);
        c_last = h[2 * i];
        w_last = h[2 * i + 1];
    }
    FDX_REQUIRE(w_last > w_first, "clock_probe_stop: no complete period inside the window");
    *mean_ghz = (double)(c_last - c_first) / (double)(w_last - w_first) * khz * 1e-6;
    *min_ghz = lo;
    *max_ghz = hi;
    return FDX_OK;
}
