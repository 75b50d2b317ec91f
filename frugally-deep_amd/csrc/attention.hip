// MultiHeadAttention core on already projected q / k / v (gfx950).
//
// Prefill shape (many query rows): scores = scale * Q K^T as one batched NT GEMM over
// (sequence, head) on fp32 MFMA, row softmax in the reference's log-sum form with an
// optional causal prefix limit, then P V as a second batched NT GEMM against V^T.
// Decode shape (one query row per sequence): a dedicated HBM-bound kernel that streams
// the token-major key / value cache once.
#include <cfloat>
#include <cmath>

#include "common.hpp"

namespace fdx {
fdx_status transpose_launch(const float* in, int batch, int rows, int cols, int64_t ld_in, int64_t in_batch, float* out);

typedef float f32x4 __attribute__((ext_vector_type(4)));

// One workgroup per (sequence, head).  Phase 1: each thread owns keys j = tid, tid+256, ...
// and dots the query (LDS) with the key row (16-byte loads).  Phase 2: block max / sum,
// probabilities back to LDS.  Phase 3: lanes run along the value depth so each cached row
// is read as one contiguous run; 256/dv key partitions are combined through LDS.
__global__ __launch_bounds__(256) void mha_decode_kernel(const float* __restrict__ q, const float* __restrict__ kc,
    const float* __restrict__ vc, float* __restrict__ out, int heads, int dk, int dv, int len, int max_len, float scale)
{
    extern __shared__ float smem[]; // [dk] query, [len] scores, [256] reduction scratch
    float* sq = smem;
    float* sp = smem + dk;
    float* red = sp + len;
    const int b = blockIdx.x / heads, h = blockIdx.x % heads, tid = threadIdx.x;
    const int64_t krow = (int64_t)heads * dk, vrow = (int64_t)heads * dv;
    for (int d = tid; d < dk; d += 256)
        sq[d] = q[(int64_t)b * krow + h * dk + d];
    __syncthreads();
    float m = -FLT_MAX;
    for (int j = tid; j < len; j += 256) {
        const float* kr = kc + ((int64_t)b * max_len + j) * krow + h * dk;
        float s = 0.f;
        if ((dk & 3) == 0) {
            for (int d = 0; d < dk; d += 4) {
                const f32x4 kv = *reinterpret_cast<const f32x4*>(kr + d);
                s += sq[d] * kv[0] + sq[d + 1] * kv[1] + sq[d + 2] * kv[2] + sq[d + 3] * kv[3];
            }
        } else {
            for (int d = 0; d < dk; ++d)
                s += sq[d] * kr[d];
        }
        s *= scale;
        sp[j] = s;
        m = fmaxf(m, s);
    }
    // block max
    for (int o = 32; o > 0; o >>= 1)
        m = fmaxf(m, __shfl_xor(m, o, 64));
    if ((tid & 63) == 0)
        red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sum = 0.f;
    for (int j = tid; j < len; j += 256)
        sum += expf(sp[j] - m);
    for (int o = 32; o > 0; o >>= 1)
        sum += __shfl_xor(sum, o, 64);
    __syncthreads();
    if ((tid & 63) == 0)
        red[tid >> 6] = sum;
    __syncthreads();
    const float ls = logf(red[0] + red[1] + red[2] + red[3]);
    for (int j = tid; j < len; j += 256) {
        const float p = expf(sp[j] - m - ls);
        sp[j] = isinf(p) ? 0.f : p;
    }
    __syncthreads();
    // P V
    const int parts = dv <= 256 ? 256 / dv : 1;
    for (int d0 = 0; d0 < dv; d0 += 256) {
        const int d = d0 + (parts > 1 ? tid % dv : tid), part = parts > 1 ? tid / dv : 0;
        float acc = 0.f;
        if (d < dv && part < parts)
            for (int j = part; j < len; j += parts)
                acc += sp[j] * vc[((int64_t)b * max_len + j) * vrow + h * dv + d];
        if (parts > 1) {
            __syncthreads();
            red[tid] = acc;
            __syncthreads();
            if (tid < dv) {
                float r = red[tid];
                for (int pidx = 1; pidx < parts; ++pidx)
                    r += red[pidx * dv + tid];
                out[(int64_t)b * vrow + h * dv + tid] = r;
            }
        } else if (d < dv) {
            out[(int64_t)b * vrow + h * dv + d] = acc;
        }
    }
}

} // namespace fdx

using namespace fdx;

extern "C" size_t fdx_mha_scratch_bytes(int batch, int heads, int t, int s, int dv)
{
    return sizeof(float) * ((size_t)batch * heads * t * s + (size_t)batch * heads * dv * s) + 256;
}

namespace fdx {
// q/k/v/out rows may be strided (ld*) and sequences apart by *_batch elements, so the key/value
// operands can live in a token-major cache and q/k/v can be column blocks of one fused projection.
fdx_status mha_prefill_strided(const float* q, int64_t ldq, int64_t q_batch, const float* k, int64_t ldk, int64_t k_batch,
    const float* v, int64_t ldv, int64_t v_batch, int batch, int t, int s, int heads, int dk, int dv, int causal,
    float* out, int64_t ldo, int64_t o_batch, void* scratch_dev)
{
    FDX_REQUIRE(q && k && v && out && scratch_dev, "mha_prefill: null pointer");
    FDX_REQUIRE(batch > 0 && t > 0 && s > 0 && heads > 0 && dk > 0 && dv > 0, "mha_prefill: bad shape");
    FDX_REQUIRE(!causal || s >= t, "mha_prefill: causal attention needs at least as many keys as queries");
    FDX_REQUIRE((int64_t)batch * heads <= 65535, "mha_prefill: batch * heads too large");
    float* scores = static_cast<float*>(scratch_dev);
    float* vt = scores + (((size_t)batch * heads * t * s + 3) & ~(size_t)3);
    const int64_t v_row = (int64_t)heads * dv;
    // 1 / sqrt(key_dim) applied to the scores after the product (multi_head_attention_layer.hpp:91-93)
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    fdx_gemm_batch bt {};
    bt.batch = batch * heads;
    bt.inner = heads;
    bt.a_outer = q_batch; bt.a_inner = dk;
    bt.b_outer = k_batch; bt.b_inner = dk;
    bt.c_outer = (int64_t)heads * t * s; bt.c_inner = (int64_t)t * s;
    fdx_status st = fdx_gemm_bias_act_f32(q, ldq, k, ldk, t, s, dk, scale, nullptr, 0, nullptr, nullptr, scores, s, &bt);
    if (st != FDX_OK)
        return st;
    st = fdx_softmax_f32(scores, (int64_t)batch * heads * t, s, causal ? t : 0, causal ? s - t : 0, scores);
    if (st != FDX_OK)
        return st;
    st = transpose_launch(v, batch, s, (int)v_row, ldv, v_batch, vt); // [b][s][H*dv] -> [b][H*dv][s]
    if (st != FDX_OK)
        return st;
    bt.a_outer = (int64_t)heads * t * s; bt.a_inner = (int64_t)t * s;
    bt.b_outer = v_row * s; bt.b_inner = (int64_t)dv * s;
    bt.c_outer = o_batch; bt.c_inner = dv;
    return fdx_gemm_bias_act_f32(scores, s, vt, s, t, dv, s, 1.0f, nullptr, 0, nullptr, nullptr, out, ldo, &bt);
}
}

extern "C" fdx_status fdx_mha_prefill_f32(const float* q, const float* k, const float* v, int batch, int t, int s,
    int heads, int dk, int dv, int causal, float* out, void* scratch_dev)
{
    const int64_t qk = (int64_t)heads * dk, vr = (int64_t)heads * dv;
    return fdx::mha_prefill_strided(q, qk, t * qk, k, qk, s * qk, v, vr, s * vr, batch, t, s, heads, dk, dv, causal, out, vr,
        t * vr, scratch_dev);
}

extern "C" fdx_status fdx_mha_decode_f32(const float* q, const float* k_cache, const float* v_cache, int batch, int heads,
    int dk, int dv, int len, int max_len, float* out)
{
    FDX_REQUIRE(q && k_cache && v_cache && out, "mha_decode: null pointer");
    FDX_REQUIRE(batch > 0 && heads > 0 && dk > 0 && dv > 0 && len > 0 && len <= max_len, "mha_decode: bad shape");
    const size_t smem = sizeof(float) * ((size_t)dk + len + 256);
    FDX_REQUIRE(smem <= 64 * 1024, "mha_decode: context length %d exceeds the single-pass kernel's LDS budget", len);
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    profile_begin();
    hipLaunchKernelGGL(mha_decode_kernel, dim3(batch * heads), dim3(256), smem, stream(), q, k_cache, v_cache, out, heads, dk,
        dv, len, max_len, scale);
    profile_end("mha_decode_f32", 4.0 * batch * heads * (double)len * dk,
        4.0 * ((double)batch * len * heads * (dk + dv) + (double)batch * heads * (dk + dv)));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
