// Two pointwise convolutions in a row as one launch, gfx950:
//     y = act1(W1 . [a | b] + bias1 + residual)        (written out: later layers read it)
//     z = act2(W2 . y + bias2)                         (written out)
// -- the tail of one residual block (1x1 convolution + Add + ReLU, include/fdeep/layers/conv_2d_layer.hpp:52-56,
// add_layer.hpp:20-29, relu_layer.hpp:40-46) and the 1x1 convolution that opens the next block.  As two launches the wide
// tensor y (four times the channels of a and z in a bottleneck block) is written once and read twice, by the next
// convolution and by the next Add; here the second convolution takes it from the workgroup's LDS, and memory sees it
// written once and read once.
//
// A workgroup of four waves (2 x 2) owns blocks of 64 pixels.  Per block:
//   * the 64 x K input rows go to LDS once (K = channels of a, plus those of b where the first convolution sums two
//     inputs -- b may be read at a stride, as the shortcut branch of a block that changes the resolution);
//   * for each tile of 64 output channels of y: the product on 32x32x2 fp32 MFMA, a wave per 32 x 32 piece, the filter
//     fragments straight from memory in the order the lanes take them (packed at load: one contiguous kilobyte per wave
//     and load, requested a chunk of 64 input channels ahead); bias, residual and activation per 16-byte row piece; the
//     finished piece is stored and left in the wave's LDS rows;
//   * the tile's 64 channels are a K slice of the second product: after one barrier every wave multiplies the rows of
//     its row pair (its own piece and its neighbour's) by the matching slice of W2 into accumulators that live across
//     the tiles;
//   * after the last tile: bias2, act2, store z.
// Nothing is exchanged between workgroups.
#include <cstring>
#include <mutex>

#include "common.hpp"
#include "igemm_params.hpp"

namespace fdx {

typedef unsigned u32x4c __attribute__((ext_vector_type(4)));

struct ChainParams {
    const float* a;        // [M][K1], rows lda floats apart
    int64_t lda;
    int K1;
    const float* b;        // optional second input of the first convolution: pixel (y * s2y, x * s2x) of an [H2][W2][C2] map
    int K2, H2, W2, C2, s2y, s2x, OH, OW; // K2 = 0: none; OH / OW: the map the M rows are pixels of
    const float* w1;       // packed, see fdx::chain_pack_first
    const float* bias1;    // [N1] or null
    const float* residual; // [M][N1] or null
    float* y;              // [M][N1]
    int N1;
    Act act1;
    const float* w2;       // packed, see fdx::chain_pack_second
    const float* bias2;    // [N2] or null
    float* z;              // [M][N2]
    Act act2;
    int M;
    uint32_t a_bytes, b_bytes, w1_bytes, w2_bytes, y_bytes, z_bytes, bias1_bytes, bias2_bytes;
};

constexpr int CH_BM = 64;      // pixels per block
constexpr int CH_SCR = 36;     // floats per scratch row (32 + padding)
constexpr uint32_t CH_OOB = 0x80000000u;

// KC = K / 64 (1 or 2), NB2 = N2 / 64 (1 or 2)
template <int KC, int NB2>
__global__ __launch_bounds__(256, 2) void pw_chain_kernel(ChainParams p)
{
    constexpr int K = KC * 64, AS = K + 4, PPT = K / 16; // A pieces (16 bytes) per thread and block
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* a_blk = lds;             // [64][AS]
    float* scr = lds + CH_BM * AS;  // [4 waves][32][CH_SCR]
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1, fr = lane & 31, fh = lane >> 5;
    const __amdgpu_buffer_rsrc_t srd_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.a), 0, (int)p.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.K2 ? p.b : p.a), 0,
        p.K2 ? (int)p.b_bytes : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_w1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.w1), 0, (int)p.w1_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_w2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.w2), 0, (int)p.w2_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_y = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, (int)p.y_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_z = __builtin_amdgcn_make_buffer_rsrc(p.z, 0, (int)p.z_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual ? p.residual : p.y), 0,
        p.residual ? (int)p.y_bytes : 0, 0x00020000);
    // without a bias the extent is empty and the loads answer zeros
    const __amdgpu_buffer_rsrc_t srd_b1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.bias1 ? p.bias1 : p.a), 0,
        (int)p.bias1_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_b2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.bias2 ? p.bias2 : p.a), 0,
        (int)p.bias2_bytes, 0x00020000);

    const int row_blocks = (p.M + CH_BM - 1) / CH_BM, n_tiles = p.N1 / 64;
    float* ws = scr + wave * 32 * CH_SCR; // this wave's scratch rows
    const int srow = lane >> 3, scol = (lane & 7) * 4; // a lane's place in a pass over the scratch: 8 rows x 8 pieces

    // filter fragments of (tile nt, chunk c) of the first product for this wave's 32 columns: 8 pieces of 16 bytes
    auto request_w1 = [&](f32x4 (&dst)[8], int nt, int c) {
        const uint32_t base = (uint32_t)(((nt * 2 + wn) * (K / 8) + c * 8) * 64 + lane) * 16u;
#pragma unroll
        for (int k8 = 0; k8 < 8; ++k8)
            dst[k8] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_w1, (int)(base + (uint32_t)k8 * 1024u), 0, 0));
    };

    // the input rows of a block: this thread's pieces (rows beyond M answer zeros)
    f32x4 piece[PPT];
    auto request_rows = [&](int m0) {
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            const int q = t + i * 256, r = q / (K / 4), kq = q - r * (K / 4), m = m0 + r;
            uint32_t off = CH_OOB;
            const bool second = kq * 4 >= p.K1;
            if (m < p.M) {
                if (!second) {
                    off = (uint32_t)((int64_t)m * p.lda) * 4u + (uint32_t)kq * 16u;
                } else {
                    const int img = m / (p.OH * p.OW), rm = m - img * (p.OH * p.OW);
                    const int oy = rm / p.OW, ox = rm - oy * p.OW;
                    off = (uint32_t)(((img * p.H2 + oy * p.s2y) * p.W2 + ox * p.s2x) * p.C2) * 4u + (uint32_t)(kq * 4 - p.K1) * 4u;
                }
            }
            const f32x4 va = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_a, (int)(second ? CH_OOB : off), 0, 0));
            const f32x4 vb = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, (int)(second ? off : CH_OOB), 0, 0));
            piece[i] = second ? vb : va;
        }
    };
    // bias and residual pieces of a tile's epilogue, requested before its product
    auto request_epilogue = [&](int m0, int nt, f32x4& bias4, f32x4 (&rr)[4]) {
        const int n = nt * 64 + wn * 32 + scol;
        bias4 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_b1, nt < n_tiles ? n * 4 : (int)CH_OOB, 0, 0));
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int m = m0 + wm * 32 + ps * 8 + srow;
            const uint32_t off = (m < p.M && nt < n_tiles) ? (uint32_t)((int64_t)m * p.N1 + n) * 4u : CH_OOB;
            rr[ps] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_res, (int)off, 0, 0));
        }
    };
    for (int rb = blockIdx.x; rb < row_blocks; rb += gridDim.x) {
        const int m0 = rb * CH_BM;
        request_rows(m0);
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            const int q = t + i * 256, r = q / (K / 4), kq = q - r * (K / 4);
            *reinterpret_cast<f32x4*>(&a_blk[r * AS + kq * 4]) = piece[i];
        }
        f32x4 w1a[8], w1b[8];
        request_w1(w1a, 0, 0);
        __syncthreads();

        f32x16 acc2[NB2];
#pragma unroll
        for (int j = 0; j < NB2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc2[j][e] = 0.f;

        // one tile of 64 channels of y; `cur` holds the fragments of its first chunk, `nxt` is free
        auto do_tile = [&](int nt, f32x4 (&cur)[8], f32x4 (&nxt)[8]) {
            const int n = nt * 64 + wn * 32 + scol; // this lane's four channels in the row passes
            uint32_t yoff[4];
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                const int m = m0 + wm * 32 + ps * 8 + srow;
                yoff[ps] = m < p.M ? (uint32_t)((int64_t)m * p.N1 + n) * 4u : CH_OOB;
            }
            f32x4 bias4, rr[4];
            request_epilogue(m0, nt, bias4, rr);
            // the slice of W2 that meets this tile's channels
            f32x4 w2f[NB2][8];
#pragma unroll
            for (int j = 0; j < NB2; ++j) {
                const uint32_t base = (uint32_t)(((nt * (NB2 * 2) + wn * NB2 + j) * 8) * 64 + lane) * 16u;
#pragma unroll
                for (int k8 = 0; k8 < 8; ++k8)
                    w2f[j][k8] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_w2, (int)(base + (uint32_t)k8 * 1024u), 0, 0));
            }
            // the fragments that follow `cur`: this tile's second chunk, or the next tile's first (beyond the last tile the
            // offsets lie behind the filter and the loads answer zeros)
            if (KC == 2)
                request_w1(nxt, nt, 1);
            else
                request_w1(nxt, nt + 1, 0);
            __builtin_amdgcn_sched_barrier(0);

            f32x16 acc1;
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc1[e] = 0.f;
            // (the row fragments are read from LDS one group of four MFMAs ahead: read right in front of their use, as the
            // scheduler would have it, every group waits out the LDS latency with the matrix pipe drained)
            auto chunk = [&](const f32x4 (&wf)[8], int c) {
                const float* arow = &a_blk[(wm * 32 + fr) * AS + c * 64 + fh * 4];
                f32x4 af[2];
                af[0] = *reinterpret_cast<const f32x4*>(arow);
#pragma unroll
                for (int k8 = 0; k8 < 8; ++k8) {
                    if (k8 < 7)
                        af[(k8 + 1) & 1] = *reinterpret_cast<const f32x4*>(arow + (k8 + 1) * 8);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(af[k8 & 1][e], wf[k8][e], acc1, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            chunk(cur, 0);
            if (KC == 2) {
                __builtin_amdgcn_sched_barrier(0);
                request_w1(cur, nt + 1, 0); // `cur` is free again: the next tile finds its first chunk there
                __builtin_amdgcn_sched_barrier(0);
                chunk(nxt, 1);
            }

            // ---- the tile's epilogue: accumulators -> this wave's scratch rows -> 16-byte row pieces
#pragma unroll
            for (int e = 0; e < 16; ++e)
                ws[(8 * (e >> 2) + 4 * fh + (e & 3)) * CH_SCR + fr] = acc1[e];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            f32x4 done[4];
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(&ws[(ps * 8 + srow) * CH_SCR + scol]);
                float r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    r[e] = v[e] + bias4[e] + rr[ps][e];
                apply_act_block(r, p.act1);
                done[ps] = f32x4 { r[0], r[1], r[2], r[3] };
            }
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                *reinterpret_cast<f32x4*>(&ws[(ps * 8 + srow) * CH_SCR + scol]) = done[ps]; // the second product's operand
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4c, done[ps]), srd_y, (int)yoff[ps], 0, 0);
            }
            __syncthreads(); // the neighbour's piece of the row pair is complete

            // ---- this tile's K slice of the second product
            {
                auto xrow = [&](int k8) {
                    return reinterpret_cast<const f32x4*>(&scr[((wm * 2 + (k8 >> 2)) * 32 + fr) * CH_SCR + (k8 & 3) * 8 + fh * 4]);
                };
                f32x4 xf[2];
                xf[0] = *xrow(0);
#pragma unroll
                for (int k8 = 0; k8 < 8; ++k8) {
                    if (k8 < 7)
                        xf[(k8 + 1) & 1] = *xrow(k8 + 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < NB2; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc2[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xf[k8 & 1][e], w2f[j][k8][e], acc2[j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __syncthreads(); // before the next epilogue overwrites the scratch rows
        };

        for (int nt = 0; nt < n_tiles; nt += 2) { // (the tile count is even)
            do_tile(nt, w1a, w1b);
            if (KC == 2)
                do_tile(nt + 1, w1a, w1b);
            else
                do_tile(nt + 1, w1b, w1a);
        }

        // ---- z: bias2, act2, store
#pragma unroll
        for (int j = 0; j < NB2; ++j) {
            const int n2 = (wn * NB2 + j) * 32 + scol;
            const f32x4 bias4 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_b2, n2 * 4, 0, 0));
#pragma unroll
            for (int e = 0; e < 16; ++e)
                ws[(8 * (e >> 2) + 4 * fh + (e & 3)) * CH_SCR + fr] = acc2[j][e];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                const int m = m0 + wm * 32 + ps * 8 + srow;
                const f32x4 v = *reinterpret_cast<const f32x4*>(&ws[(ps * 8 + srow) * CH_SCR + scol]);
                float r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    r[e] = v[e] + bias4[e];
                apply_act_block(r, p.act2);
                const f32x4 o = { r[0], r[1], r[2], r[3] };
                const uint32_t off = m < p.M ? (uint32_t)((int64_t)m * (NB2 * 64) + n2) * 4u : CH_OOB;
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4c, o), srd_z, (int)off, 0, 0);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        __syncthreads(); // the next block's rows overwrite a_blk
    }
}

static size_t chain_lds_bytes(int k) { return sizeof(float) * ((size_t)CH_BM * (size_t)(k + 4) + 4u * 32u * CH_SCR); }

// shapes the kernel covers: K = k1 + k2 input channels of the first convolution, n1 its filters, n2 those of the second
bool chain_supported(int k1, int k2, int n1, int n2)
{
    const int k = k1 + k2;
    return k1 > 0 && k1 % 4 == 0 && k2 >= 0 && k2 % 4 == 0 && (k == 64 || k == 128) && n1 >= 128 && n1 % 128 == 0 && (n2 == 64 || n2 == 128);
}

size_t chain_first_floats(int n1, int k) { return (size_t)n1 * (size_t)k; }
size_t chain_second_floats(int n1, int n2) { return (size_t)n1 * (size_t)n2; }

// w [n1][k] (row-major, the concatenated filter where there are two inputs) ->
// [n1 / 64][2][k / 8][64 lanes][4]: lane 32 * h + r of wave column wn holds w[nt * 64 + wn * 32 + r][k8 * 8 + h * 4 .. + 3]
void chain_pack_first(const float* w, int n1, int k, float* out)
{
    for (int nt = 0; nt < n1 / 64; ++nt)
        for (int wn = 0; wn < 2; ++wn)
            for (int k8 = 0; k8 < k / 8; ++k8)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < 4; ++e)
                        out[((((size_t)nt * 2 + wn) * (k / 8) + k8) * 64 + lane) * 4 + e]
                            = w[(size_t)(nt * 64 + wn * 32 + (lane & 31)) * k + k8 * 8 + (lane >> 5) * 4 + e];
}

// w [n2][n1] -> [n1 / 64][n2 / 32][8][64 lanes][4]: the slice that meets channels nt * 64 .. + 63 of the first product, lane
// 32 * h + r of column piece j holds w[j * 32 + r][nt * 64 + k8 * 8 + h * 4 .. + 3]
void chain_pack_second(const float* w, int n1, int n2, float* out)
{
    for (int nt = 0; nt < n1 / 64; ++nt)
        for (int j = 0; j < n2 / 32; ++j)
            for (int k8 = 0; k8 < 8; ++k8)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < 4; ++e)
                        out[((((size_t)nt * (n2 / 32) + j) * 8 + k8) * 64 + lane) * 4 + e]
                            = w[(size_t)(j * 32 + (lane & 31)) * n1 + nt * 64 + k8 * 8 + (lane >> 5) * 4 + e];
}

static bool al16c(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

template <int KC, int NB2>
static fdx_status chain_launch_as(const ChainParams& p)
{
    const size_t lds = chain_lds_bytes(KC * 64);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(pw_chain_kernel<KC, NB2>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)chain_lds_bytes(KC * 64));
    if (attr != hipSuccess) {
        set_error("conv1x1_chain: the kernel's LDS request was refused");
        return FDX_ERR_UNSUPPORTED;
    }
    static const int resident = [] {
        int dev = 0, per_cu = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess
            || hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, pw_chain_kernel<KC, NB2>, 256, chain_lds_bytes(KC * 64)) != hipSuccess)
            return 0;
        return per_cu * prop.multiProcessorCount;
    }();
    if (resident <= 0) {
        set_error("conv1x1_chain: no occupancy figure for the kernel");
        return FDX_ERR_HIP;
    }
    const int row_blocks = (p.M + CH_BM - 1) / CH_BM;
    const dim3 grid((unsigned)(row_blocks < resident ? row_blocks : resident));
    hipLaunchKernelGGL((pw_chain_kernel<KC, NB2>), grid, dim3(256), lds, stream(), p);
    return FDX_OK;
}

// y = act1(W1 . [a | b] + bias1 + residual), z = act2(W2 . y + bias2) over n * oh * ow pixels; w1 / w2 packed by
// chain_pack_first / chain_pack_second.  b (k2 > 0) is read at pixel (y * s2y, x * s2x) of an [n][h2][w2][c2] tensor.
// FDX_ERR_UNSUPPORTED, with nothing launched, for shapes or sizes the kernel does not cover.
fdx_status conv1x1_chain_launch(const float* a, int n, int oh, int ow, int k1, const float* b, int h2, int w2, int c2, int s2y, int s2x,
    int k2, const float* w1, const float* bias1, const float* residual, const fdx_act* act1, int n1, float* y, const float* w2p,
    const float* bias2, const fdx_act* act2, int n2, float* z)
{
    FDX_REQUIRE(a && w1 && w2p && y && z && n > 0 && oh > 0 && ow > 0 && (k2 == 0 || b), "conv1x1_chain: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act1);
    FDX_REQUIRE_EPILOGUE_ACT(act2);
    const int64_t m = (int64_t)n * oh * ow;
    if (!chain_supported(k1, k2, n1, n2) || m >= (1LL << 31) || m * n1 * 4 >= (1LL << 31) || m * k1 * 4 >= (1LL << 31) || !al16c(a) || !al16c(w1)
        || !al16c(w2p) || !al16c(y) || !al16c(z) || (b && !al16c(b)) || (bias1 && !al16c(bias1)) || (bias2 && !al16c(bias2))
        || (residual && !al16c(residual))) {
        set_error("conv1x1_chain: shape or size outside the kernel");
        return FDX_ERR_UNSUPPORTED;
    }
    ChainParams p;
    std::memset(&p, 0, sizeof p);
    p.a = a; p.lda = k1; p.K1 = k1; p.a_bytes = (uint32_t)(m * k1 * 4);
    p.OH = oh; p.OW = ow;
    if (k2 > 0) {
        FDX_REQUIRE(h2 > 0 && w2 > 0 && c2 >= k2 && c2 % 4 == 0 && s2y > 0 && s2x > 0 && (int64_t)(oh - 1) * s2y < h2 && (int64_t)(ow - 1) * s2x < w2,
            "conv1x1_chain: bad second input");
        if ((int64_t)n * h2 * w2 * c2 * 4 >= (1LL << 31)) {
            set_error("conv1x1_chain: second input beyond 2 GiB");
            return FDX_ERR_UNSUPPORTED;
        }
        p.b = b; p.K2 = k2; p.H2 = h2; p.W2 = w2; p.C2 = c2; p.s2y = s2y; p.s2x = s2x;
        p.b_bytes = (uint32_t)((int64_t)n * h2 * w2 * c2 * 4);
    }
    p.w1 = w1; p.bias1 = bias1; p.residual = residual; p.y = y; p.N1 = n1; p.act1 = make_act(act1);
    p.w2 = w2p; p.bias2 = bias2; p.z = z; p.act2 = make_act(act2);
    p.M = (int)m;
    p.w1_bytes = (uint32_t)(chain_first_floats(n1, k1 + k2) * 4);
    p.w2_bytes = (uint32_t)(chain_second_floats(n1, n2) * 4);
    p.y_bytes = (uint32_t)(m * n1 * 4);
    p.z_bytes = (uint32_t)(m * n2 * 4);
    p.bias1_bytes = bias1 ? (uint32_t)n1 * 4u : 0u;
    p.bias2_bytes = bias2 ? (uint32_t)n2 * 4u : 0u;
    profile_begin();
    fdx_status st;
    const int kc = (k1 + k2) / 64, nb2 = n2 / 64;
    if (kc == 1 && nb2 == 1)
        st = chain_launch_as<1, 1>(p);
    else if (kc == 2 && nb2 == 1)
        st = chain_launch_as<2, 1>(p);
    else if (kc == 1 && nb2 == 2)
        st = chain_launch_as<1, 2>(p);
    else
        st = chain_launch_as<2, 2>(p);
    if (st != FDX_OK)
        return st;
    profile_end("conv1x1_chain_f32", 2.0 * (double)m * n1 * ((double)k1 + k2 + n2),
        4.0 * ((double)m * (k1 + k2 + n1 * (residual ? 2.0 : 1.0) + n2) + (double)n1 * (k1 + k2 + n2)));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

} // namespace fdx
