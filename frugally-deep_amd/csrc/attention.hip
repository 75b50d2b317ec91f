// MultiHeadAttention core on already projected q / k / v (gfx950).
//
// Prefill shape (many query rows): one fused pass for head depths 32 / 64 / 128 (scores, softmax
// and P V on fp32 MFMA with the probabilities kept in registers); any other depth runs as
// scores = scale * Q K^T (one batched NT GEMM over (sequence, head)), row softmax in the
// reference's log-sum form with an optional causal prefix limit, then P V as a second batched
// NT GEMM against V^T.
// Decode shape (one query row per sequence): a dedicated HBM-bound kernel that streams
// the token-major key / value cache once.
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdlib>

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

// ---- fused prefill attention: scores, softmax and P V in one pass, nothing but the output written --------------------
//
// One workgroup = 128 query rows of one (sequence, head), one wave = 32 of them; keys / values pass through LDS in
// tiles of 64.  The products are taken transposed on the 32x32x2 fp32 MFMA: S^T = K Q^T puts a query on a lane
// (column) and keys on the accumulator registers, so the running maximum, the running sum and the rescaling of the
// flash-attention recurrence are per-lane scalars, and the probabilities P^T are already laid out as the B operand of
// O^T = V^T P^T -- they never leave the registers.  The contraction index of either product may be visited in any
// order as long as both operands agree, which is what lets the accumulator layout (keys 8j + 4*half + i in register
// 4j + i) feed the second product directly.
//
// Softmax as the reference takes it (include/fdeep/tensor.hpp:1165-1192) is exp(x - max - log(sum exp(x - max)));
// here the running maximum replaces max and the division by the running sum comes last, which agrees to rounding.
struct FlashParams {
    const float* q; int64_t ldq, q_batch;
    const float* k; int64_t ldk, k_batch;
    const float* v; int64_t ldv, v_batch;
    float* out; int64_t ldo, o_batch;
    int t, s, heads, causal;
    float scale;
};

typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int DK, int DV>
__global__ __launch_bounds__(256) void flash_prefill_kernel(FlashParams p)
{
    constexpr int KS = DK + 4;  // LDS row strides: 16-byte fragment reads along a key row stay conflict-free
    constexpr int VS = DV + 8;  // lanes read along the depth; rows 4 apart (the two lane halves) fall on disjoint banks
    constexpr int KL = DK / 16, VL = DV / 16; // 16-byte loads per thread for a 64-row tile
    __shared__ __attribute__((aligned(16))) float ks[64 * KS];
    __shared__ __attribute__((aligned(16))) float vs[64 * VS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, half = lane >> 5;
    const int b = blockIdx.y / p.heads, h = blockIdx.y % p.heads;
    const int q_first = blockIdx.x * 128;
    const int query = q_first + wave * 32 + c;
    const bool q_ok = query < p.t;
    const int shift = p.s - p.t; // causal: query i sees keys 0 .. i + shift

    // this lane's half of its query row: depth 8u + 4*half .. + 3, the same split the key fragments use
    f32x4 qreg[DK / 8];
    {
        const float* qrow = p.q + (int64_t)b * p.q_batch + (int64_t)(q_ok ? query : 0) * p.ldq + h * DK + 4 * half;
#pragma unroll
        for (int u = 0; u < DK / 8; ++u)
            qreg[u] = q_ok ? *reinterpret_cast<const f32x4*>(qrow + 8 * u) : f32x4 { 0.f, 0.f, 0.f, 0.f };
    }

    // keys this workgroup needs: all of them, or up to the last one its last query may see
    int s_end = p.s;
    if (p.causal) {
        const int q_last = (q_first + 128 < p.t ? q_first + 128 : p.t) - 1;
        s_end = q_last + shift + 1 < p.s ? q_last + shift + 1 : p.s;
    }
    const int tiles = (s_end + 63) / 64;
    const int wave_q_last = q_first + wave * 32 + 31;

    const float* kbase = p.k + (int64_t)b * p.k_batch + h * DK;
    const float* vbase = p.v + (int64_t)b * p.v_batch + h * DV;
    f32x4 kst[KL], vst[VL];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int idx = tid + 256 * i, row = idx / (DK / 4), c4 = idx % (DK / 4);
            kst[i] = j0 + row < p.s ? *reinterpret_cast<const f32x4*>(kbase + (int64_t)(j0 + row) * p.ldk + 4 * c4)
                                     : f32x4 { 0.f, 0.f, 0.f, 0.f };
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int idx = tid + 256 * i, row = idx / (DV / 4), c4 = idx % (DV / 4);
            vst[i] = j0 + row < p.s ? *reinterpret_cast<const f32x4*>(vbase + (int64_t)(j0 + row) * p.ldv + 4 * c4)
                                     : f32x4 { 0.f, 0.f, 0.f, 0.f };
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int idx = tid + 256 * i, row = idx / (DK / 4), c4 = idx % (DK / 4);
            *reinterpret_cast<f32x4*>(&ks[row * KS + 4 * c4]) = kst[i];
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int idx = tid + 256 * i, row = idx / (DV / 4), c4 = idx % (DV / 4);
            *reinterpret_cast<f32x4*>(&vs[row * VS + 4 * c4]) = vst[i];
        }
    };

    f32x16 oacc[DV / 32];
#pragma unroll
    for (int d = 0; d < DV / 32; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            oacc[d][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    if (tiles > 0)
        fetch(0);
    for (int tile = 0; tile < tiles; ++tile) {
        const int j0 = tile * 64;
        __syncthreads(); // every wave is done with the previous tile
        stage();
        __syncthreads();
        if (tile + 1 < tiles)
            fetch(j0 + 64); // in flight while this tile is worked on
        if (p.causal && j0 > wave_q_last + shift)
            continue; // nothing in this tile is visible to any of this wave's queries (wave-uniform)

        // S^T tile: 64 keys x 32 queries
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                sacc[kb][e] = 0.f;
#pragma unroll
            for (int u = 0; u < DK / 8; ++u) {
                const f32x4 kf = *reinterpret_cast<const f32x4*>(&ks[(kb * 32 + c) * KS + 8 * u + 4 * half]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qreg[u][e], sacc[kb], 0, 0, 0);
            }
        }
        // scale, mask, running maximum
        const int key_limit = p.causal ? (query + shift < p.s - 1 ? query + shift : p.s - 1) : p.s - 1;
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int key = j0 + kb * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                const float sv = key <= key_limit ? sacc[kb][e] * p.scale : -INFINITY;
                sacc[kb][e] = sv;
                mx = fmaxf(mx, sv);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        // a query that has seen no key yet (rows past the end of the sequence) keeps zeros instead of NaNs
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float corr = expf(m_run - m_use);
        float rs = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float pv = __expf(sacc[kb][e] - m_use);
                sacc[kb][e] = pv;
                rs += pv;
            }
        rs += __shfl_xor(rs, 32, 64);
        l_run = l_run * corr + rs;
        m_run = m_new;
#pragma unroll
        for (int d = 0; d < DV / 32; ++d)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                oacc[d][e] *= corr;
        // O^T += V^T P^T
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float* vrow = &vs[(kb * 32 + 8 * (e >> 2) + 4 * half + (e & 3)) * VS + c];
#pragma unroll
                for (int d = 0; d < DV / 32; ++d)
                    oacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * d], sacc[kb][e], oacc[d], 0, 0, 0);
            }
    }

    if (q_ok) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        float* orow = p.out + (int64_t)b * p.o_batch + (int64_t)query * p.ldo + h * DV + 4 * half;
#pragma unroll
        for (int d = 0; d < DV / 32; ++d)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 o = { oacc[d][4 * g] * inv, oacc[d][4 * g + 1] * inv, oacc[d][4 * g + 2] * inv, oacc[d][4 * g + 3] * inv };
                *reinterpret_cast<f32x4*>(orow + 32 * d + 8 * g) = o;
            }
    }
}

template <int DK, int DV>
static void flash_launch(const FlashParams& p, int batch)
{
    const dim3 grid((unsigned)((p.t + 127) / 128), (unsigned)(batch * p.heads));
    hipLaunchKernelGGL((flash_prefill_kernel<DK, DV>), grid, dim3(256), 0, stream(), p);
}

static bool flash_enabled()
{
    static const bool on = [] {
        const char* e = std::getenv("FDX_FLASH");
        return !(e && e[0] == '0');
    }();
    return on;
}

// true when the fused kernel took the call
static bool flash_prefill(const FlashParams& p, int batch, int dk, int dv)
{
    if (!flash_enabled())
        return false;
    auto aligned = [](const void* ptr, int64_t ld, int64_t bs) {
        return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0 && (ld & 3) == 0 && (bs & 3) == 0;
    };
    if (!aligned(p.q, p.ldq, p.q_batch) || !aligned(p.k, p.ldk, p.k_batch) || !aligned(p.v, p.ldv, p.v_batch)
        || !aligned(p.out, p.ldo, p.o_batch))
        return false;
    profile_begin();
    if (dk == 64 && dv == 64)
        flash_launch<64, 64>(p, batch);
    else if (dk == 32 && dv == 32)
        flash_launch<32, 32>(p, batch);
    else if (dk == 128 && dv == 128)
        flash_launch<128, 128>(p, batch);
    else
        return false;
    const double pairs = p.causal ? (double)p.t * (p.s - p.t) + 0.5 * (double)p.t * (p.t + 1) : (double)p.t * p.s;
    profile_end("mha_flash_f32", 2.0 * batch * p.heads * pairs * (dk + dv),
        4.0 * batch * p.heads * ((double)p.t * (dk + dv) + (double)p.s * (dk + dv)));
    return true;
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
    // 1 / sqrt(key_dim) applied to the scores after the product (multi_head_attention_layer.hpp:91-93)
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    {
        FlashParams fp { q, ldq, q_batch, k, ldk, k_batch, v, ldv, v_batch, out, ldo, o_batch, t, s, heads, causal, scale };
        if (flash_prefill(fp, batch, dk, dv)) {
            FDX_LAUNCH_CHECK();
            return FDX_OK;
        }
    }
    float* scores = static_cast<float*>(scratch_dev);
    float* vt = scores + (((size_t)batch * heads * t * s + 3) & ~(size_t)3);
    const int64_t v_row = (int64_t)heads * dv;
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
