// Row-streaming GEMM for short K (K <= 128): C[M][N] = act(alpha * A[M][K] * B[N][K]^T + bias + residual).
// Included by igemm.hip inside namespace fdx.  One more form of the product behind convolve with a 1x1 filter
// (include/fdeep/convolution.hpp:398-429) and dense_layer::apply_impl (include/fdeep/layers/dense_layer.hpp:76-86).
//
// The pointwise convolutions that widen a tensor (K = 16..128 input channels, N = 96..960 outputs) are one or two K
// slabs of arithmetic around a large output: the tiled kernel spends its time in tile set-up, LDS staging and barriers
// while the memory system waits for stores.  Here every wave works on its own, without LDS and without barriers: it
// takes 32 rows of A straight into MFMA operand registers (a lane's fragment is 16 contiguous bytes of its row, a wave's
// load covers whole rows), walks the 32-column groups of the output with the B fragments read from L2 (B is a few KB to
// a few hundred KB and every wave reads all of it), and stores each 32x32 result from the accumulator layout (one store
// writes two 128-byte row pieces).  All accesses go through buffer resources: rows beyond M, columns beyond N and k
// blocks beyond K get an out-of-range offset instead of a branch, and a row that is shorter than K (a_valid_k: the
// padded pointwise case, where a row laps into the next pixel) ends at the extent like on the tiled path.
#pragma once

struct PwStreamParams {
    GemmParams g;
    uint32_t a_bytes, b_bytes, c_bytes;
};

template <int K8> // k blocks of 8 held in registers: K <= 8 * K8
__global__ __launch_bounds__(256) void pw_stream_kernel(PwStreamParams q)
{
    const GemmParams& p = q.g;
    constexpr uint32_t OOB = 0x80000000u;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fr = lane & 31, fh = lane >> 5;
    const __amdgpu_buffer_rsrc_t srd_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.A), 0, (int)q.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.B), 0, (int)q.b_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_c = __builtin_amdgcn_make_buffer_rsrc(p.C, 0, (int)q.c_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_r = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual ? p.residual : p.C), 0,
        (int)q.c_bytes, 0x00020000);
    const int kb = p.K / 8, CT = (p.N + 31) / 32;
    const int tiles = (p.M + 31) / 32, wave_count = (int)gridDim.x * 4;
    for (int tile = (int)blockIdx.x * 4 + wave; tile < tiles; tile += wave_count) {
        const int row = tile * 32 + fr;
        f32x4 af[K8];
#pragma unroll
        for (int k8 = 0; k8 < K8; ++k8) {
            const uint32_t vo = (row < p.M && k8 < kb) ? ((uint32_t)row * (uint32_t)p.lda + k8 * 8 + fh * 4) * 4u : OOB;
            af[k8] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_a, (int)vo, 0, 0));
        }
        // 32x32 accumulator layout: element e of lane l is row 8*(e/4) + 4*(l/32) + e%4, column l%32
        uint32_t row_off[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int m = tile * 32 + 8 * (e >> 2) + 4 * fh + (e & 3);
            row_off[e] = m < p.M ? (uint32_t)m * (uint32_t)p.ldc * 4u : OOB;
        }
        for (int ct = 0; ct < CT; ++ct) {
            const int ncol = ct * 32 + fr;
            const bool n_ok = ncol < p.N;
            f32x4 bf[K8];
#pragma unroll
            for (int k8 = 0; k8 < K8; ++k8) {
                const uint32_t vo = (n_ok && k8 < kb) ? ((uint32_t)ncol * (uint32_t)p.ldb + k8 * 8 + fh * 4) * 4u : OOB;
                bf[k8] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, (int)vo, 0, 0));
            }
            const float bcol = (p.bias && n_ok) ? p.bias[ncol] : 0.f;
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[e] = 0.f;
#pragma unroll
            for (int k8 = 0; k8 < K8; ++k8)
                if (k8 < kb) { // uniform
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[k8][e], bf[k8][e], acc, 0, 0, 0);
                }
            float v[16];
            uint32_t off[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                off[e] = (n_ok && row_off[e] != OOB) ? row_off[e] + (uint32_t)ncol * 4u : OOB;
                v[e] = acc[e] * p.alpha + bcol;
            }
            if (p.residual) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    v[e] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srd_r, (int)off[e], 0, 0));
            }
            apply_act_block(v, p.act);
#pragma unroll
            for (int e = 0; e < 16; ++e)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[e]), srd_c, (int)off[e], 0, 16); // agent scope: written through to memory, nothing left dirty in L2 at the kernel's end
        }
    }
}

// whether the row-streaming kernel can run this problem (GEMM form only)
static bool pw_stream_ok(const GemmParams& p, bool conv, int batch, int64_t a_bytes, int64_t b_bytes)
{
    const int64_t c_bytes = ((int64_t)(p.M - 1) * p.ldc + p.N) * 4;
    return !conv && batch == 1 && p.K % 8 == 0 && p.K <= 128 && p.lda % 4 == 0 && p.ldb % 4 == 0 && !p.bias_per_row
        && (reinterpret_cast<uintptr_t>(p.A) & 15) == 0 && (reinterpret_cast<uintptr_t>(p.B) & 15) == 0 && a_bytes < (1LL << 31)
        && b_bytes < (1LL << 31) && c_bytes < (1LL << 31) && (int64_t)p.M * p.lda < (1LL << 29) && (int64_t)p.M * p.ldc < (1LL << 29);
}

static void pw_stream_launch(const GemmParams& p, int64_t a_bytes, int64_t b_bytes, hipStream_t s)
{
    PwStreamParams q;
    q.g = p;
    q.a_bytes = (uint32_t)a_bytes;
    q.b_bytes = (uint32_t)b_bytes;
    q.c_bytes = (uint32_t)(((int64_t)(p.M - 1) * p.ldc + p.N) * 4);
    const int tiles = (p.M + 31) / 32;
    const int want = (tiles + 3) / 4;
#define FDX_PWS(K8_)                                                                                         \
    {                                                                                                        \
        const int resident = resident_workgroups(pw_stream_kernel<K8_>, 256);                                \
        hipLaunchKernelGGL(pw_stream_kernel<K8_>, dim3((unsigned)(want < resident ? want : resident)), dim3(256), 0, s, q); \
    }
    if (p.K <= 32)
        FDX_PWS(4)
    else if (p.K <= 64)
        FDX_PWS(8)
    else
        FDX_PWS(16)
#undef FDX_PWS
}
