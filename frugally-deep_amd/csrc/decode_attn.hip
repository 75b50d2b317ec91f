// Decode attention for the common head shape (key_dim = value_dim = 64, at most 256 cached
// positions): one query row per (sequence, head) against the token-major key / value cache.
//
// The kernel is one memory round trip: every lane issues all of its key AND value loads
// (16 bytes each, sixteen lanes per cached row so a wave touches four whole rows per load)
// before anything is used; the values do not depend on the softmax, so they travel while the
// scores are reduced.  Scores stay in registers; max / sum / output reductions use wave
// shuffles and ONE small LDS exchange between the four waves.  Softmax weights equal the
// reference's exp(x - m - log(sum)) (include/fdeep/tensor.hpp:1165-1192) up to rounding; the
// scale multiplies the scores after the dot product (layers/multi_head_attention_layer.hpp:91-93).
#include <cfloat>
#include <cmath>

#include "common.hpp"
#include "skinny.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void mha_decode_fast_kernel(const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ kc, const float* __restrict__ vc, float* __restrict__ out, int heads,
    const int* __restrict__ len_dev, int max_len, float scale)
{
    __shared__ float red[4], red_sum[4];
    __shared__ float osum[4][64];
    const int tid = threadIdx.x, part = tid & 15, slot = tid >> 4, wave = tid >> 6;
    const int b = blockIdx.x / heads, h = blockIdx.x % heads;
    const int len = *len_dev + 1;
    const int64_t row = (int64_t)heads * 64;
    const float* kbase = kc + (int64_t)b * max_len * row + h * 64 + part * 4;
    const float* vbase = vc + (int64_t)b * max_len * row + h * 64 + part * 4;
    f32x4 kv[16], vv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const int j = slot + 16 * u;
        kv[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
        vv[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
        if (j < len) {
            kv[u] = *reinterpret_cast<const f32x4*>(kbase + (int64_t)j * row);
            vv[u] = *reinterpret_cast<const f32x4*>(vbase + (int64_t)j * row);
        }
    }
    const f32x4 qv = *reinterpret_cast<const f32x4*>(q + (int64_t)b * ldq + h * 64 + part * 4);

    float sc[16];
    float m = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        float s = qv[0] * kv[u][0] + qv[1] * kv[u][1] + qv[2] * kv[u][2] + qv[3] * kv[u][3];
        s += __shfl_xor(s, 8, 64);
        s += __shfl_xor(s, 4, 64);
        s += __shfl_xor(s, 2, 64);
        s += __shfl_xor(s, 1, 64);
        sc[u] = slot + 16 * u < len ? s * scale : -FLT_MAX;
        m = fmaxf(m, sc[u]);
    }
    // Each wave finishes its own quarter of the keys against its OWN maximum (the other slots of the wave sit 16 and
    // 32 lanes away): probabilities, their sum and the weighted values.  The four quarters then meet once in LDS and
    // are rescaled to the common maximum, exp(m_w - m) each -- one barrier instead of one per reduction.  The result
    // is the reference's exp(x - m - log(sum)) weighting up to rounding.
    m = fmaxf(m, __shfl_xor(m, 16, 64));
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float sum = 0.f;
    f32x4 acc = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const float pr = slot + 16 * u < len ? expf(sc[u] - m) : 0.f;
        sum += pr;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            acc[e] += pr * vv[u][e];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        acc[e] += __shfl_xor(acc[e], 16, 64);
        acc[e] += __shfl_xor(acc[e], 32, 64);
    }
    if ((tid & 63) < 16) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            osum[wave][part * 4 + e] = acc[e];
    }
    if ((tid & 63) == 0) {
        red[wave] = m;
        red_sum[wave] = sum;
    }
    __syncthreads();
    if (tid < 64) {
        const float mm = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        float f[4], denom = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            f[w] = expf(red[w] - mm); // a wave without a visible key has m_w = -FLT_MAX: weight 0
            denom += f[w] * red_sum[w];
            o += f[w] * osum[w][tid];
        }
        out[(int64_t)b * row + h * 64 + tid] = o / denom;
    }
}

// true if the fast kernel covers this shape; launches it
bool mha_decode_fast_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch, int heads,
    int dk, int dv, const int* len_dev, int max_len, hipStream_t s)
{
    if (dk != 64 || dv != 64 || max_len > 256 || ldq % 4 != 0)
        return false;
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    hipLaunchKernelGGL(mha_decode_fast_kernel, dim3(batch * heads), dim3(256), 0, s, q, ldq, kc, vc, out, heads, len_dev, max_len, scale);
    return true;
}

} // namespace fdx
