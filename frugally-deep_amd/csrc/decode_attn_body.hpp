// Body of the decode attention for the common head shape, shared by the attention kernel and the kernel that also
// applies the output projection (both in decode_attn.hip).  Included inside namespace fdx after f32x4 and gptr are defined.
#pragma once

struct MhaDecodeShared {
    float red[4], red_sum[4];
    float osum[4][64];
    float oval[64]; // KEEP: the head's output row for the code that follows in the same workgroup
};

// The work of one (sequence, head) item by 256 threads.  KEEP: the 64 output values stay in sh.oval (valid after the
// caller's next barrier) instead of going to `out`.
// after_loads() runs once every key / value / query load has been issued and before the first of them is used: the place
// where a caller requests operands of its own that do not depend on the attention result.
template <bool KEEP, typename AfterLoads>
__device__ __forceinline__ void mha_decode_fast_body(const float* __restrict__ q, int64_t ldq, const float* __restrict__ kc,
    const float* __restrict__ vc, float* __restrict__ out, int heads, const int* __restrict__ len_dev, int max_len, float scale,
    int item, int tid, bool active, MhaDecodeShared& sh, AfterLoads after_loads)
{
    float* red = sh.red;
    float* red_sum = sh.red_sum;
    float (*osum)[64] = sh.osum;
    const int part = tid & 15, slot = tid >> 4, wave = (tid >> 6) & 3;
    const int b = item / heads, h = item % heads;
    const int len = active ? *as_global(len_dev) + 1 : 0;
    const int64_t row = (int64_t)heads * 64;
    const gptr<const float> kbase = as_global(kc) + (int64_t)b * max_len * row + h * 64 + part * 4;
    const gptr<const float> vbase = as_global(vc) + (int64_t)b * max_len * row + h * 64 + part * 4;
    f32x4 kv[16], vv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const int j = slot + 16 * u;
        kv[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
        vv[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
        if (j < len) {
            kv[u] = *reinterpret_cast<gptr<const f32x4>>(kbase + (int64_t)j * row);
            vv[u] = *reinterpret_cast<gptr<const f32x4>>(vbase + (int64_t)j * row);
        }
    }
    const f32x4 qv = active ? *reinterpret_cast<gptr<const f32x4>>(as_global(q) + (int64_t)b * ldq + h * 64 + part * 4) : f32x4 { 0.f, 0.f, 0.f, 0.f };
    after_loads();

    float sc[16];
    float m = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        float s = qv[0] * kv[u][0] + qv[1] * kv[u][1] + qv[2] * kv[u][2] + qv[3] * kv[u][3];
        s = row16_sum(s);
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
        const float pr = slot + 16 * u < len ? __expf(sc[u] - m) : 0.f; // as the prefill kernel: the hardware exponential, relative error ~1e-7
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
    if (active && (tid & 63) < 16) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            osum[wave][part * 4 + e] = acc[e];
    }
    if (active && (tid & 63) == 0) {
        red[wave] = m;
        red_sum[wave] = sum;
    }
    __syncthreads();
    if (active && tid < 64) {
        const float mm = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        float f[4], denom = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            f[w] = expf(red[w] - mm); // a wave without a visible key has m_w = -FLT_MAX: weight 0
            denom += f[w] * red_sum[w];
            o += f[w] * osum[w][tid];
        }
        if (KEEP)
            sh.oval[tid] = o / denom;
        else
            as_global(out)[(int64_t)b * row + h * 64 + tid] = o / denom;
    }
}

