// A whole inverted-residual block as one launch, gfx950: 1x1 expansion -> depthwise 3x3 -> 1x1 projection.
//
// The expanded tensor of such a block is several times wider than its input and output (six times in MobileNetV2)
// and, computed layer by layer, crosses HBM two to four times.  Here it never leaves the CU: a wave owns a tile of
// 4 x 8 output pixels; for one slab of 32 expanded channels at a time it
//   1. multiplies the input pixels under the tile (with the stencil's one-pixel frame: 6 x 10 of them at stride 1,
//      9 x 17 at stride 2) by the slab's 32 rows of the expansion filter on fp32 MFMA, adds the bias, applies the
//      activation and leaves the result in its own LDS rows -- zero where the pixel lies outside the image, because
//      that is what the depthwise convolution's padding reads (the padded value is not expand(0)),
//   2. runs the 3x3 stencil over those LDS rows (one lane per run of four output pixels and four channels), applies
//      the second activation and writes the 32 x 32 result as the A operand of
//   3. the projection: multiplied by the slab's 32 columns of the 1x1 filter on MFMA into accumulators that live in
//      registers across the slabs.
// Bias, residual and activation of the projection are applied before the only store.  Both 1x1 filters sit in LDS for
// the lifetime of the workgroup; waves never synchronise with each other inside the loop.  The frame pixels are
// expanded once per tile that touches them (1.9x the expansion's multiply-adds at stride 1, 1.2x at stride 2), the
// price of not writing the expanded tensor: HBM traffic is the block's input and output.
//
// The reference computes the three layers one after the other: convolve (include/fdeep/convolution.hpp:398-429), the
// activation, depthwise_convolve (include/fdeep/depthwise_convolution.hpp:21-99), the activation, convolve, Add.
#include <cstring>
#include <map>
#include <mutex>

#include "common.hpp"
#include "igemm_params.hpp"

// a size the kernel's 32-bit offsets do not cover: not an error of the caller, who has the layer-by-layer launches
#define FDX_FUSED_LIMIT(cond, ...)                                                                        \
    do {                                                                                                  \
        if (!(cond)) {                                                                                    \
            fdx::set_error(__VA_ARGS__);                                                                  \
            return FDX_ERR_UNSUPPORTED;                                                                   \
        }                                                                                                 \
    } while (0)

namespace fdx {

struct IrbParams {
    const float* in;       // [n][h][w][cin]
    const float* exp_w;    // [ce][cin]
    const float* exp_b;    // [ce] or null
    const float* dw_w;     // [3][3][ce]
    const float* dw_b;     // [ce] or null
    const float* pw_w;     // [N][ce]
    const float* pw_b;     // [N] or null
    const float* residual; // like out, or null
    float* out;            // [n][oh][ow][N]
    int n, h, w, ce, pad_top, pad_left, oh, ow, N;
    int tiles_x, tiles_y, tiles; // tiles of 4 x 8 output pixels per row band / per image column, and all of them
    int ce_pad;                  // ce rounded up to the channel slab
    uint32_t in_bytes, out_bytes; // extents of input and output / residual (below 2^31)
    Act act_exp, act_dw, act_out;
    // stem form: the first layer is an ek x ek convolution (stride es, padding ept / epl) on the image `in`
    // [n][ih][iw][ic] with ek * ek * ic <= 32; h and w are then the extents of that convolution's output and exp_w is
    // [ce][ek][ek][ic]
    int ih, iw, ic, ek, es, ept, epl;
};

constexpr int IRB_TH = 4, IRB_TW = 8, IRB_TX = 4; // output tile of a wave; pixels per stencil run
constexpr int IRB_KC = 32;                         // expanded channels per slab
constexpr int IRB_LS = IRB_KC + 4;                 // padded LDS row of a slab: conflict-free 128-bit accesses
constexpr int IRB_NP = 64;                         // widest projection: two 32-column MFMA tiles

// floats of LDS one wave needs for its expanded slab and the projection's A operand
constexpr int irb_wave_floats(int stride)
{
    const int pin = ((IRB_TH - 1) * stride + 3) * ((IRB_TW - 1) * stride + 3);
    return ((pin + 31) / 32) * 32 * IRB_LS + 32 * IRB_LS;
}

// ReLU with an upper bound and nothing else (ReLU6, plain ReLU: threshold 0, slope 0) is one median-of-three per value;
// every other activation takes the general block form.  (Below the threshold the general form returns slope * x = -0.0
// where this returns +0.0; the two compare equal and multiply alike.)
__device__ __forceinline__ bool irb_is_clamp(const Act& a)
{
    return a.kind == FDX_ACT_RELU && a.negative_slope == 0.f && a.threshold == 0.f;
}
template <int COUNT>
__device__ __forceinline__ void irb_act(float (&v)[COUNT], const Act& a, bool clamp)
{
    if (clamp) {
#pragma unroll
        for (int z = 0; z < COUNT; ++z)
            v[z] = __builtin_amdgcn_fmed3f(v[z], 0.f, a.max_value);
    } else
        apply_act_block(v, a);
}

// KIN = input channels / 8, CT = 32-column tiles of the projection, NW = waves per workgroup.  STEM: the first layer is
// a small convolution on an image of a few channels instead of a 1x1 convolution (the first block of MobileNet-like
// networks: 3x3 / 2 on RGB, depthwise 3x3, 1x1 projection); its taps, (filter row, filter column, channel) = k < 32,
// take the place of the input channels, and the A operand is gathered from the image tap by tap.
template <int STRIDE, int CT, int KIN, int NW, bool STEM>
__global__ __launch_bounds__(NW * 64) void irb_kernel(IrbParams p)
{
    constexpr int TH = IRB_TH, TW = IRB_TW, TX = IRB_TX, KC = IRB_KC, LS = IRB_LS;
    constexpr int RH = (TH - 1) * STRIDE + 3, RW = (TW - 1) * STRIDE + 3, PIN = RH * RW, RB = (PIN + 31) / 32;
    constexpr int COLS = (TX - 1) * STRIDE + 3, CIN = KIN * 8, WS = CIN + 4;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int fr = lane & 31, fh = lane >> 5;
    const int ce = p.ce, BS = p.ce_pad + 4;
    float* Bs = lds;                       // projection filter [CT * 32][ce_pad + 4]
    float* We = Bs + CT * 32 * BS;         // expansion filter [ce_pad][CIN + 4]
    float* Wd = We + p.ce_pad * WS;        // depthwise filter [9][ce_pad], then the expansion bias [ce_pad] and the depthwise bias [ce_pad]
    float* Be = Wd + 9 * p.ce_pad;
    float* Bd = Be + p.ce_pad;
    float* Es = Bd + p.ce_pad + wave * irb_wave_floats(STRIDE); // this wave's expanded slab [RB * 32][LS]
    float* As = Es + RB * 32 * LS;         // this wave's depthwise result [32][LS]

    for (int idx = t; idx < CT * 32 * (p.ce_pad / 4); idx += NW * 64) {
        const int nrow = idx / (p.ce_pad / 4), ch = (idx % (p.ce_pad / 4)) * 4;
        f32x4 w4 = { 0.f, 0.f, 0.f, 0.f };
        if (nrow < p.N && ch < ce)
            w4 = *reinterpret_cast<const f32x4*>(p.pw_w + (int64_t)nrow * ce + ch);
        *reinterpret_cast<f32x4*>(&Bs[nrow * BS + ch]) = w4;
    }
    if (STEM) {
        const int taps = p.ek * p.ek * p.ic;
        for (int idx = t; idx < p.ce_pad * CIN; idx += NW * 64) {
            const int row = idx / CIN, k = idx - row * CIN;
            We[row * WS + k] = (row < ce && k < taps) ? p.exp_w[(int64_t)row * taps + k] : 0.f;
        }
    } else {
        for (int idx = t; idx < p.ce_pad * KIN * 2; idx += NW * 64) {
            const int row = idx / (KIN * 2), k4 = (idx % (KIN * 2)) * 4;
            f32x4 w4 = { 0.f, 0.f, 0.f, 0.f };
            if (row < ce)
                w4 = *reinterpret_cast<const f32x4*>(p.exp_w + (int64_t)row * CIN + k4);
            *reinterpret_cast<f32x4*>(&We[row * WS + k4]) = w4;
        }
    }
    for (int idx = t; idx < 11 * p.ce_pad; idx += NW * 64) { // every per-slab operand comes from LDS: a global load per slab would stall the wave
        const int row = idx / p.ce_pad, ch = idx - row * p.ce_pad;
        float v = 0.f;
        if (ch < ce) {
            if (row < 9)
                v = p.dw_w[(int64_t)row * ce + ch];
            else if (row == 9)
                v = p.exp_b ? p.exp_b[ch] : 0.f;
            else
                v = p.dw_b ? p.dw_b[ch] : 0.f;
        }
        Wd[idx] = v;
    }
    __syncthreads();

    constexpr uint32_t OOB = 0x80000000u; // beyond any extent the host accepts
    const __amdgpu_buffer_rsrc_t srd_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.in), 0, (int)p.in_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_out = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, (int)p.out_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual ? p.residual : p.out), 0,
        (int)p.out_bytes, 0x00020000);
    const bool clamp_exp = irb_is_clamp(p.act_exp), clamp_dw = irb_is_clamp(p.act_dw), clamp_out = irb_is_clamp(p.act_out);
    const int run_local = lane >> 3, q = lane & 7; // stencil item of this lane: run of the tile, channel quad of the slab
    const int orow = run_local >> 1, xrun = run_local & 1; // the run's row in the tile and which half of the row
    // stem form: tap k = kk * 8 + fh * 4 + e of this lane in one word: bits 0-23 its byte offset from the window's
    // first tap, bits 24-26 the filter row, 27-29 the filter column, bit 31 set for a tap beyond the filter (added to
    // an offset it points outside every extent, and the load returns zero)
    uint32_t tap[KIN][4];
    if (STEM) {
        const int taps = p.ek * p.ek * p.ic, row_taps = p.ek * p.ic;
#pragma unroll
        for (int kk = 0; kk < KIN; ++kk)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k = kk * 8 + fh * 4 + e;
                const int ky = k / row_taps, rem = k - ky * row_taps;
                tap[kk][e] = k < taps ? (uint32_t)((ky * p.iw * p.ic + rem) * 4) | (uint32_t)ky << 24 | (uint32_t)(rem / p.ic) << 27 : OOB;
            }
    }
    const int wave_count = (int)gridDim.x * NW;
    // The input pixels of a tile in MFMA operand order: row block rb, row fr is region pixel rb * 32 + fr; this lane
    // holds channels kk * 8 + fh * 4 .. + 3 of it.  A pixel outside the image (or beyond the region) reads as zeros.
    // (Requesting the next tile's pixels once the last slab's expansion has freed these registers was measured: slower,
    // the longer live ranges cost more than the hidden latency gains.)
    f32x4 a[RB][KIN];
    auto request_pixels = [&](int tile) {
        const int rest = tile / p.tiles_x;
        const int tx = tile - rest * p.tiles_x;
        const int img = rest / p.tiles_y;
        const int ty = rest - img * p.tiles_y;
        const int iy0 = ty * TH * STRIDE - p.pad_top, ix0 = tx * TW * STRIDE - p.pad_left;
        const uint32_t img_off = STEM ? (uint32_t)img * (uint32_t)(p.ih * p.iw * p.ic) * 4u : (uint32_t)img * (uint32_t)(p.h * p.w * CIN) * 4u;
        if (STEM) {
            // every window of the region inside the image (most tiles): no test per tap
            const int wy0 = iy0 * p.es - p.ept, wx0 = ix0 * p.es - p.epl;
            const bool windows_inside = iy0 >= 0 && iy0 + RH <= p.h && ix0 >= 0 && ix0 + RW <= p.w && wy0 >= 0 && wx0 >= 0
                && wy0 + (RH - 1) * p.es + p.ek <= p.ih && wx0 + (RW - 1) * p.es + p.ek <= p.iw;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int pidx = rb * 32 + fr;
                const int ry = pidx / RW, rx = pidx - ry * RW;
                const int iy = iy0 + ry, ix = ix0 + rx;
                const int by = iy * p.es - p.ept, bx = ix * p.es - p.epl; // first tap of this pixel's window
                const uint32_t base = img_off + (uint32_t)((by * p.iw + bx) * p.ic * 4); // wraps below zero and back with the tap's offset
                if (windows_inside) {
#pragma unroll
                    for (int kk = 0; kk < KIN; ++kk)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t off = pidx < PIN ? base + (tap[kk][e] & 0x80FFFFFFu) : OOB;
                            a[rb][kk][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srd_in, (int)off, 0, 0));
                        }
                } else {
                    const bool ok = pidx < PIN && iy >= 0 && iy < p.h && ix >= 0 && ix < p.w;
#pragma unroll
                    for (int kk = 0; kk < KIN; ++kk)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int yy = by + (int)((tap[kk][e] >> 24) & 7u), xx = bx + (int)((tap[kk][e] >> 27) & 7u);
                            const bool tap_ok = ok && yy >= 0 && yy < p.ih && xx >= 0 && xx < p.iw;
                            const uint32_t off = tap_ok ? base + (tap[kk][e] & 0x80FFFFFFu) : OOB;
                            a[rb][kk][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srd_in, (int)off, 0, 0));
                        }
                }
            }
        } else {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int pidx = rb * 32 + fr;
                const int ry = pidx / RW, rx = pidx - ry * RW;
                const int iy = iy0 + ry, ix = ix0 + rx;
                const bool ok = pidx < PIN && iy >= 0 && iy < p.h && ix >= 0 && ix < p.w;
                const uint32_t off = ok ? img_off + (uint32_t)((iy * p.w + ix) * CIN + fh * 4) * 4u : OOB;
#pragma unroll
                for (int kk = 0; kk < KIN; ++kk)
                    a[rb][kk] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_in, (int)(off + (uint32_t)kk * 32u), 0, 0));
            }
        }
    };
    for (int tile = (int)blockIdx.x * NW + wave; tile < p.tiles; tile += wave_count) {
        request_pixels(tile);
        const int rest = tile / p.tiles_x;
        const int tx = tile - rest * p.tiles_x;
        const int img = rest / p.tiles_y;
        const int ty = rest - img * p.tiles_y;
        const int oy0 = ty * TH, ox0 = tx * TW;
        const int iy0 = oy0 * STRIDE - p.pad_top, ix0 = ox0 * STRIDE - p.pad_left;
        // which of the sixteen accumulator rows of a row block are pixels inside the image: element e of this lane is row
        // 8 * (e / 4) + 4 * fh + e % 4
        // (a tile whose whole region lies inside the image -- most of them -- needs no mask)
        const bool interior = iy0 >= 0 && iy0 + RH <= p.h && ix0 >= 0 && ix0 + RW <= p.w;
        uint32_t inside[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            uint32_t bits = 0xFFFFu;
            if (!interior) {
                bits = 0;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int pidx = rb * 32 + 8 * (e / 4) + 4 * fh + (e % 4);
                const int ry = pidx / RW, rx = pidx - ry * RW;
                const int iy = iy0 + ry, ix = ix0 + rx;
                bits |= (pidx < PIN && iy >= 0 && iy < p.h && ix >= 0 && ix < p.w) ? (1u << e) : 0u;
            }
            }
            inside[rb] = bits;
        }

        f32x16 acc[CT];
#pragma unroll
        for (int i = 0; i < CT; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][e] = 0.f;

        for (int c_base = 0; c_base < ce; c_base += KC) {
            // ---- 1. expansion of the slab: E[pixel][channel c_base + fr]
            const bool col_ok = c_base + fr < ce;
            const float be = Be[c_base + fr];
            f32x4 bf[KIN];
#pragma unroll
            for (int kk = 0; kk < KIN; ++kk)
                bf[kk] = *reinterpret_cast<const f32x4*>(&We[(c_base + fr) * WS + kk * 8 + fh * 4]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                f32x16 ex; // the accumulators start at the bias of this lane's column
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    ex[e] = be;
#pragma unroll
                for (int kk = 0; kk < KIN; ++kk)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        ex = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][kk][e], bf[kk][e], ex, 0, 0, 0);
                float v[16];
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    v[e] = ex[e];
                irb_act(v, p.act_exp, clamp_exp);
                if (interior && c_base + KC <= ce) { // nothing to mask: every pixel inside the image, every column a channel
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        Es[(rb * 32 + 8 * (e / 4) + 4 * fh + (e % 4)) * LS + fr] = v[e];
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const bool keep = col_ok && ((inside[rb] >> e) & 1u);
                        Es[(rb * 32 + 8 * (e / 4) + 4 * fh + (e % 4)) * LS + fr] = keep ? v[e] : 0.f;
                    }
                }
            }
            __builtin_amdgcn_wave_barrier(); // a wave runs its LDS accesses in order: the stencil below reads what was written above

            // ---- 2. depthwise 3x3 on the slab
            const int c0 = c_base + 4 * q;
            const bool c_ok = c0 < ce;
            f32x4 wv[9];
#pragma unroll
            for (int k = 0; k < 9; ++k)
                wv[k] = *reinterpret_cast<const f32x4*>(&Wd[k * p.ce_pad + c0]);
            const f32x4 b4 = *reinterpret_cast<const f32x4*>(&Bd[c0]);
            float o[TX * 4];
#pragma unroll
            for (int j = 0; j < TX; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    o[j * 4 + v] = b4[v];
            const float* ebase = Es + ((orow * STRIDE) * RW + xrun * TX * STRIDE) * LS + 4 * q;
#pragma unroll
            for (int fy = 0; fy < 3; ++fy) {
                f32x4 col[COLS];
#pragma unroll
                for (int k = 0; k < COLS; ++k)
                    col[k] = *reinterpret_cast<const f32x4*>(ebase + (fy * RW + k) * LS);
#pragma unroll
                for (int j = 0; j < TX; ++j)
#pragma unroll
                    for (int fx = 0; fx < 3; ++fx)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            o[j * 4 + v] += col[j * STRIDE + fx][v] * wv[fy * 3 + fx][v];
            }
            irb_act(o, p.act_dw, clamp_dw);
            // pixels beyond the image and channels beyond the last are zero rows / columns of the product's A operand
#pragma unroll
            for (int j = 0; j < TX; ++j) {
                const bool keep = c_ok && oy0 + orow < p.oh && ox0 + xrun * TX + j < p.ow;
                const f32x4 r = { keep ? o[j * 4 + 0] : 0.f, keep ? o[j * 4 + 1] : 0.f, keep ? o[j * 4 + 2] : 0.f, keep ? o[j * 4 + 3] : 0.f };
                *reinterpret_cast<f32x4*>(&As[(run_local * TX + j) * LS + 4 * q]) = r;
            }
            __builtin_amdgcn_wave_barrier();

            // ---- 3. projection of the slab
#pragma unroll
            for (int k8 = 0; k8 < KC / 8; ++k8) {
                const f32x4 af = *reinterpret_cast<const f32x4*>(&As[fr * LS + k8 * 8 + fh * 4]);
#pragma unroll
                for (int i = 0; i < CT; ++i) {
                    const f32x4 pf = *reinterpret_cast<const f32x4*>(&Bs[(i * 32 + fr) * BS + c_base + k8 * 8 + fh * 4]);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[e], pf[e], acc[i], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier(); // the next slab overwrites both LDS areas
        }

        // ---- epilogue.  Element e of lane l is tile pixel 8 * (e / 4) + 4 * (l / 32) + e % 4, i.e. output row e / 4 of
        // the tile, column 4 * (l / 32) + e % 4; accumulator column l % 32.  Elements outside the tensor get an
        // out-of-range offset: the store is dropped, the residual reads as zero.
#pragma unroll
        for (int i = 0; i < CT; ++i) {
            const int ncol = i * 32 + fr;
            const bool n_ok = ncol < p.N;
            const float bcol = (p.pw_b && n_ok) ? p.pw_b[ncol] : 0.f;
            float v[16];
            uint32_t off[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int oy = oy0 + e / 4, ox = ox0 + 4 * fh + (e % 4);
                off[e] = (n_ok && oy < p.oh && ox < p.ow) ? (uint32_t)(((img * p.oh + oy) * p.ow + ox) * p.N + ncol) * 4u : OOB;
                v[e] = acc[i][e] + bcol;
            }
            if (p.residual) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    v[e] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srd_res, (int)off[e], 0, 0));
            }
            irb_act(v, p.act_out, clamp_out);
#pragma unroll
            for (int e = 0; e < 16; ++e)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[e]), srd_out, (int)off[e], 0, 16); // agent scope: written through to memory, nothing left dirty in L2 at the kernel's end
        }
    }
}

static size_t irb_lds_bytes(int cin, int ce, int n_out, int stride, int waves)
{
    const int ce_pad = (ce + IRB_KC - 1) / IRB_KC * IRB_KC, ct = (n_out + 31) / 32;
    return sizeof(float) * ((size_t)ct * 32 * (ce_pad + 4) + (size_t)ce_pad * (cin + 4) + (size_t)11 * ce_pad + (size_t)waves * irb_wave_floats(stride));
}

// LDS a workgroup may ask for on this part (the occupancy query below refuses a launch that does not fit)
constexpr size_t kIrbLdsLimit = 160 * 1024;

// waves per workgroup: eight where the LDS allows (stride 1), else four
static int irb_waves(int cin, int ce, int n_out, int stride)
{
    if (irb_lds_bytes(cin, ce, n_out, stride, 8) <= kIrbLdsLimit)
        return 8;
    if (irb_lds_bytes(cin, ce, n_out, stride, 4) <= kIrbLdsLimit)
        return 4;
    return 0;
}

// workgroups of `kernel` that are resident at once with `lds` bytes of dynamic LDS; raises the kernel's LDS limit once
template <typename K>
static int64_t irb_resident(K kernel, int threads, size_t lds)
{
    // keyed by the kernel's address as well: the instantiations share one function type, and the dynamic LDS limit is
    // an attribute of each of them
    static std::mutex mu;
    static std::map<std::pair<const void*, size_t>, int64_t> known;
    const std::pair<const void*, size_t> key(reinterpret_cast<const void*>(kernel), lds);
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find(key);
    if (it != known.end())
        return it->second;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return known[key] = 0;
    int per_cu = 0, dev = 0;
    hipDeviceProp_t prop;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds) != hipSuccess || per_cu < 1)
        return known[key] = 0;
    const int cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) ? prop.multiProcessorCount : 256;
    return known[key] = (int64_t)per_cu * cus;
}

// Fills the tile counts and extents of `p` (pointers, image / grid sizes, channel counts and activations are set) and
// launches the instantiation for (depthwise stride, projection width, K / 8 of the first layer).
static fdx_status irb_launch(IrbParams& p, int cin, int n_out, int stride, bool stem, int64_t in_floats)
{
    p.tiles_x = (p.ow + IRB_TW - 1) / IRB_TW;
    p.tiles_y = (p.oh + IRB_TH - 1) / IRB_TH;
    FDX_FUSED_LIMIT((int64_t)p.n * p.tiles_x * p.tiles_y < (1LL << 30), "inverted_residual: too many output pixels for one launch");
    p.tiles = p.n * p.tiles_x * p.tiles_y;
    p.ce_pad = (p.ce + IRB_KC - 1) / IRB_KC * IRB_KC;
    FDX_FUSED_LIMIT(in_floats * 4 < (1LL << 31), "inverted_residual: input tensor beyond 2 GiB");
    p.in_bytes = (uint32_t)(in_floats * 4);
    FDX_FUSED_LIMIT((int64_t)p.n * p.oh * p.ow * n_out * 4 < (1LL << 31), "inverted_residual: output tensor beyond 2 GiB");
    p.out_bytes = (uint32_t)((int64_t)p.n * p.oh * p.ow * n_out * 4);
    const int ct = (n_out + 31) / 32, kin = cin / 8;
    const int nw = irb_waves(cin, p.ce, n_out, stride);
    const size_t lds = irb_lds_bytes(cin, p.ce, n_out, stride, nw);
    const int64_t want = ((int64_t)p.tiles + nw - 1) / nw;
    bool launched = false;
#define FDX_IRB_L(S_, CT_, KIN_, NW_, ST_)                                                                                \
    {                                                                                                                     \
        const int64_t resident = irb_resident(irb_kernel<S_, CT_, KIN_, NW_, ST_>, NW_ * 64, lds);                        \
        if (resident > 0) {                                                                                               \
            const unsigned grid = (unsigned)(want < resident ? want : resident);                                          \
            hipLaunchKernelGGL((irb_kernel<S_, CT_, KIN_, NW_, ST_>), dim3(grid), dim3(NW_ * 64), lds, stream(), p);      \
            launched = true;                                                                                              \
        }                                                                                                                 \
    }
#define FDX_IRB_W(S_, CT_, KIN_, ST_)                                                                                     \
    {                                                                                                                     \
        if (nw == 8)                                                                                                      \
            FDX_IRB_L(S_, CT_, KIN_, 8, ST_)                                                                              \
        else                                                                                                              \
            FDX_IRB_L(S_, CT_, KIN_, 4, ST_)                                                                              \
    }
#define FDX_IRB_K(S_, CT_)                                                                                                \
    {                                                                                                                     \
        if (stem)                                                                                                         \
            FDX_IRB_W(S_, CT_, 4, true)                                                                                   \
        else if (kin == 2)                                                                                                \
            FDX_IRB_W(S_, CT_, 2, false)                                                                                  \
        else if (kin == 3)                                                                                                \
            FDX_IRB_W(S_, CT_, 3, false)                                                                                  \
        else                                                                                                              \
            FDX_IRB_W(S_, CT_, 4, false)                                                                                  \
    }
    if (stride == 1) {
        if (ct == 1) FDX_IRB_K(1, 1) else FDX_IRB_K(1, 2)
    } else {
        if (ct == 1) FDX_IRB_K(2, 1) else FDX_IRB_K(2, 2)
    }
#undef FDX_IRB_K
#undef FDX_IRB_W
#undef FDX_IRB_L
    if (!launched) {
        set_error("inverted_residual: the kernel's LDS request was refused");
        return FDX_ERR_UNSUPPORTED;
    }
    return FDX_OK;
}

static bool al16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

} // namespace fdx

using namespace fdx;

extern "C" int fdx_inverted_residual_supported(int cin, int ce, int n_out, int stride)
{
    return (cin == 16 || cin == 24 || cin == 32) && ce > 0 && ce % 4 == 0 && n_out > 0 && n_out <= IRB_NP && (stride == 1 || stride == 2)
        && irb_waves(cin, ce, n_out, stride) > 0;
}

extern "C" fdx_status fdx_inverted_residual_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* exp_weights_ec,
    const float* exp_bias, const fdx_act* exp_act, int ce, const float* dw_weights_hwc, const float* dw_bias, int stride, int pad_top,
    int pad_left, int out_h, int out_w, const fdx_act* dw_act, const float* pw_weights_nc, const float* pw_bias, int n_out,
    const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && exp_weights_ec && dw_weights_hwc && pw_weights_nc && out, "inverted_residual: null pointer");
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0, "inverted_residual: bad shape");
    if (!fdx_inverted_residual_supported(cin, ce, n_out, stride)) {
        set_error("inverted_residual: needs 16, 24 or 32 input channels, expanded channels %% 4 == 0 that fit the LDS, at most %d output "
                  "channels and stride 1 or 2", IRB_NP);
        return FDX_ERR_UNSUPPORTED;
    }
    FDX_REQUIRE_EPILOGUE_ACT(exp_act);
    FDX_REQUIRE_EPILOGUE_ACT(dw_act);
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(al16(in) && al16(exp_weights_ec) && al16(dw_weights_hwc) && al16(pw_weights_nc) && (!dw_bias || al16(dw_bias)),
        "inverted_residual: operands must be 16-byte aligned");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0 && (int64_t)(out_h - 1) * stride - pad_top < h && (int64_t)(out_w - 1) * stride - pad_left < w,
        "inverted_residual: output size does not fit the input");
    IrbParams p;
    std::memset(&p, 0, sizeof p);
    p.in = in; p.exp_w = exp_weights_ec; p.exp_b = exp_bias; p.dw_w = dw_weights_hwc; p.dw_b = dw_bias; p.pw_w = pw_weights_nc;
    p.pw_b = pw_bias; p.residual = residual; p.out = out;
    p.n = n; p.h = h; p.w = w; p.ce = ce; p.pad_top = pad_top; p.pad_left = pad_left; p.oh = out_h; p.ow = out_w; p.N = n_out;
    p.act_exp = make_act(exp_act);
    p.act_dw = make_act(dw_act);
    p.act_out = make_act(act);
    profile_begin();
    const fdx_status st = irb_launch(p, cin, n_out, stride, false, (int64_t)n * h * w * cin);
    if (st != FDX_OK)
        return st;
    const double pix_in = (double)n * h * w, pix_out = (double)n * out_h * out_w;
    profile_end("inverted_residual_f32", 2.0 * pix_in * cin * ce + 2.0 * pix_out * ce * n_out,
        4.0 * (pix_in * cin + pix_out * n_out * (residual ? 2.0 : 1.0) + (double)ce * (cin + 9.0 + n_out)));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

extern "C" int fdx_stem_block_supported(int ic, int ek, int ce, int n_out, int stride)
{
    return ic > 0 && ek > 0 && ek <= 5 && ek * ek * ic <= 32 && ce > 0 && ce % 4 == 0 && n_out > 0 && n_out <= IRB_NP && (stride == 1 || stride == 2)
        && irb_waves(32, ce, n_out, stride) > 0;
}

extern "C" fdx_status fdx_stem_block_nhwc_f32(const float* in, int n, int ih, int iw, int ic, const float* conv_weights_nk,
    const float* conv_bias, const fdx_act* conv_act, int ce, int ek, int conv_stride, int conv_pad_top, int conv_pad_left, int h, int w,
    const float* dw_weights_hwc, const float* dw_bias, int stride, int pad_top, int pad_left, int out_h, int out_w, const fdx_act* dw_act,
    const float* pw_weights_nc, const float* pw_bias, int n_out, const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && conv_weights_nk && dw_weights_hwc && pw_weights_nc && out, "stem_block: null pointer");
    FDX_REQUIRE(n > 0 && ih > 0 && iw > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0 && conv_stride > 0, "stem_block: bad shape");
    if (!fdx_stem_block_supported(ic, ek, ce, n_out, stride)) {
        set_error("stem_block: needs a square filter with at most 32 taps (rows x columns x channels), convolution channels %% 4 == 0 "
                  "that fit the LDS, at most %d output channels and depthwise stride 1 or 2", IRB_NP);
        return FDX_ERR_UNSUPPORTED;
    }
    FDX_REQUIRE_EPILOGUE_ACT(conv_act);
    FDX_REQUIRE_EPILOGUE_ACT(dw_act);
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(al16(dw_weights_hwc) && al16(pw_weights_nc) && (!dw_bias || al16(dw_bias)), "stem_block: depthwise and projection operands "
        "must be 16-byte aligned");
    FDX_REQUIRE(conv_pad_top >= 0 && conv_pad_left >= 0 && conv_pad_top < 256 && conv_pad_left < 256
            && (int64_t)(h - 1) * conv_stride - conv_pad_top < ih && (int64_t)(w - 1) * conv_stride - conv_pad_left < iw,
        "stem_block: the convolution's output size does not fit the image");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0 && (int64_t)(out_h - 1) * stride - pad_top < h && (int64_t)(out_w - 1) * stride - pad_left < w,
        "stem_block: output size does not fit the convolution's output");
    FDX_FUSED_LIMIT((int64_t)iw * ic * ek * 4 < (1LL << 24), "stem_block: image rows too long");
    IrbParams p;
    std::memset(&p, 0, sizeof p);
    p.in = in; p.exp_w = conv_weights_nk; p.exp_b = conv_bias; p.dw_w = dw_weights_hwc; p.dw_b = dw_bias; p.pw_w = pw_weights_nc;
    p.pw_b = pw_bias; p.residual = residual; p.out = out;
    p.n = n; p.h = h; p.w = w; p.ce = ce; p.pad_top = pad_top; p.pad_left = pad_left; p.oh = out_h; p.ow = out_w; p.N = n_out;
    p.ih = ih; p.iw = iw; p.ic = ic; p.ek = ek; p.es = conv_stride; p.ept = conv_pad_top; p.epl = conv_pad_left;
    p.act_exp = make_act(conv_act);
    p.act_dw = make_act(dw_act);
    p.act_out = make_act(act);
    profile_begin();
    const fdx_status st = irb_launch(p, 32, n_out, stride, true, (int64_t)n * ih * iw * ic);
    if (st != FDX_OK)
        return st;
    const double pix_mid = (double)n * h * w, pix_out = (double)n * out_h * out_w;
    profile_end("stem_block_f32", 2.0 * pix_mid * ek * ek * ic * ce + 2.0 * pix_out * ce * n_out,
        4.0 * ((double)n * ih * iw * ic + pix_out * n_out * (residual ? 2.0 : 1.0) + (double)ce * (ek * ek * ic + 9.0 + n_out)));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
