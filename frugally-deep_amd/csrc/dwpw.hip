// Depthwise 3x3 convolution fused into the pointwise (1x1) convolution that consumes it, gfx950.
//
// An inverted-residual block writes its widest tensor twice and reads it twice: the expanded activations go
// expand -> HBM -> depthwise -> HBM -> projection.  Here the depthwise result never reaches memory: a wave
// computes the depthwise outputs of a tile of pixels for a slab of channels straight into LDS (the A operand),
// multiplies them by the matching slab of the 1x1 filter on fp32 MFMA, and walks the channel slabs with the
// projection's accumulators in registers.  Traffic: input once (plus the cache-served 3x3 neighbourhood), output
// once.
//
// The reference computes the two layers one after the other: depthwise_convolve
// (include/fdeep/depthwise_convolution.hpp:21-99), the activation layer, convolve (include/fdeep/convolution.hpp:398-429);
// SeparableConv2D is the same pair without anything in between (include/fdeep/layers/separable_conv_2d_layer.hpp:26-55).
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

struct DwPwParams {
    const float* in;
    const float* dw_w;  // [3][3][c]
    const float* dw_b;  // [c] or null
    const float* pw_w;  // [N][c]
    const float* pw_b;  // [N] or null
    const float* residual; // like out, or null
    float* out;         // [n][oh][ow][N]
    int n, h, w, c, pad_top, pad_left, oh, ow, N;
    int xt;             // runs per output row
    int runs;           // n * oh * xt (the host keeps it below 2^31: 32-bit index arithmetic in the kernel)
    int c_pad;          // c rounded up to the channel slab
    uint32_t in_bytes;  // extent of the input tensor (below 2^31)
    uint32_t out_bytes; // extent of the output tensor and of the residual (below 2^31)
    Act act1, act2;
};

constexpr int DWPW_NP = 96;   // widest projection: three 32-column MFMA tiles
constexpr int DWPW_TX = 4;    // output pixels per run
constexpr int DWPW_KC = 32;   // channels per slab
constexpr int DWPW_AS = DWPW_KC + 4; // padded LDS row: conflict-free 128-bit fragment reads

// Every wave works on its own: a tile of 8 runs of 4 consecutive output pixels (32 GEMM rows), one stencil item
// (run, 4 channels) per lane and 32-channel slab, its own A slab in LDS, its own accumulators.  Only the 1x1 filter is
// shared: the whole [N][c] matrix sits in LDS for the lifetime of the workgroup (zero-padded to whole slabs and column
// tiles), loaded once.  Without workgroup barriers in the loop the waves of a CU drift apart and cover each other's
// load latency, as in the stand-alone depthwise kernel.
// B_LDS = false: the filter is too large for the LDS; every wave then takes its B fragments of a slab straight from
// memory (the filter is a few hundred KB, read by every tile: it stays in L2), requested ahead of the slab's taps.
template <int STRIDE, int CT, bool B_LDS>
__global__ __launch_bounds__(256) void dwpw_kernel(DwPwParams p)
{
    constexpr int TX = DWPW_TX, COLS = (TX - 1) * STRIDE + 3, KC = DWPW_KC, AS = DWPW_AS;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int fr = lane & 31, fh = lane >> 5;
    const int c = p.c, BS = p.c_pad + 4;
    float* Bs = lds;                                  // [CT * 32][c_pad + 4] (B_LDS only)
    float* As = lds + (B_LDS ? CT * 32 * BS : 0) + wave * (32 * AS); // this wave's [32][KC + 4]

    if (B_LDS) {
        for (int idx = t; idx < CT * 32 * (p.c_pad / 4); idx += 256) {
            const int nrow = idx / (p.c_pad / 4), ch = (idx % (p.c_pad / 4)) * 4;
            f32x4 w4 = { 0.f, 0.f, 0.f, 0.f };
            if (nrow < p.N && ch < c)
                w4 = *reinterpret_cast<const f32x4*>(p.pw_w + (int64_t)nrow * c + ch);
            *reinterpret_cast<f32x4*>(&Bs[nrow * BS + ch]) = w4;
        }
        __syncthreads();
    }
    const __amdgpu_buffer_rsrc_t srd_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.pw_w), 0, p.N * c * 4, 0x00020000);

    constexpr uint32_t OOB = 0x80000000u; // beyond any extent the host accepts
    const __amdgpu_buffer_rsrc_t srd_out = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, (int)p.out_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual ? p.residual : p.out), 0,
        (int)p.out_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.in), 0, (int)p.in_bytes, 0x00020000);
    const int run_local = lane >> 3, q = lane & 7; // stencil item of this lane: run of the tile, channel quad of the slab
    const int tiles = (p.runs + 7) / 8;
    const int wave_count = (int)gridDim.x * 4;
    for (int tile = (int)blockIdx.x * 4 + wave; tile < tiles; tile += wave_count) {
        const int run = tile * 8 + run_local;
        const bool run_ok = run < p.runs;
        int ox0 = 0, oy = 0, img = 0;
        if (run_ok) {
            const unsigned rest = (unsigned)run / (unsigned)p.xt;
            ox0 = (int)((unsigned)run - rest * (unsigned)p.xt) * TX;
            img = (int)(rest / (unsigned)p.oh);
            oy = (int)(rest - (unsigned)img * (unsigned)p.oh);
        }
        // input taps through a buffer resource: a tap outside the image (or a lane without a run) gets an offset beyond
        // the extent, and the load returns zeros without a branch
        const uint32_t img_off = (uint32_t)img * (uint32_t)(p.h * p.w * c) * 4u;
        const int ix0 = ox0 * STRIDE - p.pad_left;
        const int iy0 = oy * STRIDE - p.pad_top;
        uint32_t col_ok = 0; // bit k: column ix0 + k lies inside the image
#pragma unroll
        for (int k = 0; k < COLS; ++k)
            col_ok |= (run_ok && ix0 + k >= 0 && ix0 + k < p.w) ? (1u << k) : 0u;
        uint32_t row_off[3];
#pragma unroll
        for (int fy = 0; fy < 3; ++fy) {
            const int iy = iy0 + fy;
            row_off[fy] = (iy >= 0 && iy < p.h) ? img_off + (uint32_t)((iy * p.w + ix0) * c) * 4u : OOB;
        }

        f32x16 acc[CT];
#pragma unroll
        for (int i = 0; i < CT; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][e] = 0.f;

        for (int c_base = 0; c_base < c; c_base += KC) {
            // (filter fragments of this slab first: loads return in order, and the product needs them last)
            f32x4 bw[B_LDS ? 1 : CT * (KC / 8)];
            if (!B_LDS) {
#pragma unroll
                for (int i = 0; i < CT; ++i)
#pragma unroll
                    for (int k8 = 0; k8 < KC / 8; ++k8) {
                        const int nrow = i * 32 + fr, ch = c_base + k8 * 8 + fh * 4;
                        const uint32_t vo = (nrow < p.N && ch < c) ? (uint32_t)(nrow * c + ch) * 4u : OOB;
                        bw[i * (KC / 8) + k8] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_w, (int)vo, 0, 0));
                    }
            }
            const int c0 = c_base + 4 * q;
            const bool c_ok = c0 < c;
            const int cw = c_ok ? c0 : 0; // filter taps and bias of a quad beyond the last channel: any valid address, unused
            f32x4 wv[9];
#pragma unroll
            for (int k = 0; k < 9; ++k)
                wv[k] = *reinterpret_cast<const f32x4*>(p.dw_w + (int64_t)k * c + cw);
            const f32x4 b4 = p.dw_b ? *reinterpret_cast<const f32x4*>(p.dw_b + cw) : f32x4 { 0.f, 0.f, 0.f, 0.f };
            float o[TX * 4];
#pragma unroll
            for (int j = 0; j < TX; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    o[j * 4 + v] = b4[v];
#pragma unroll
            for (int fy = 0; fy < 3; ++fy) {
                f32x4 col[COLS];
#pragma unroll
                for (int k = 0; k < COLS; ++k) {
                    const uint32_t vo = (c_ok && ((col_ok >> k) & 1u) && row_off[fy] != OOB) ? row_off[fy] + (uint32_t)(k * c + c0) * 4u : OOB;
                    col[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_in, (int)vo, 0, 0));
                }
#pragma unroll
                for (int j = 0; j < TX; ++j)
#pragma unroll
                    for (int fx = 0; fx < 3; ++fx)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            o[j * 4 + v] += col[j * STRIDE + fx][v] * wv[fy * 3 + fx][v];
            }
            apply_act_block(o, p.act1);
            // rows of pixels beyond the row end, of runs beyond the last and of channels beyond the last are zero (an
            // activation may map 0 to something else)
#pragma unroll
            for (int j = 0; j < TX; ++j) {
                const bool keep = run_ok && c_ok && ox0 + j < p.ow;
                const f32x4 r = { keep ? o[j * 4 + 0] : 0.f, keep ? o[j * 4 + 1] : 0.f, keep ? o[j * 4 + 2] : 0.f, keep ? o[j * 4 + 3] : 0.f };
                *reinterpret_cast<f32x4*>(&As[(run_local * TX + j) * AS + 4 * q]) = r;
            }
            // (the previous slab's fragment reads are behind this wave: a wave runs its LDS accesses in order)
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int k8 = 0; k8 < KC / 8; ++k8) {
                const f32x4 af = *reinterpret_cast<const f32x4*>(&As[fr * AS + k8 * 8 + fh * 4]);
#pragma unroll
                for (int i = 0; i < CT; ++i) {
                    const f32x4 bf = B_LDS ? *reinterpret_cast<const f32x4*>(&Bs[(i * 32 + fr) * BS + c_base + k8 * 8 + fh * 4])
                                           : bw[B_LDS ? 0 : i * (KC / 8) + k8];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[e], bf[e], acc[i], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }

        // ---- epilogue.  32x32 accumulator layout: element e of lane l is row 8*(e/4) + 4*(l/32) + e%4, column l%32;
        // a row is pixel e%4 of run 2*(e/4) + l/32 of the tile.
        // Output and residual through buffer resources too: an element outside the tensor (column beyond N, pixel beyond
        // the row end, run beyond the last) gets an out-of-range offset, which the hardware drops (store) or answers with
        // zero (load) -- no branch per element.
        // this lane's four runs are two apart: one division for the first, carries for the rest
        int line0 = (int)((unsigned)(tile * 8 + fh) / (unsigned)p.xt); // img * oh + oy
        int xr0 = tile * 8 + fh - line0 * p.xt;
        uint32_t pix_off[4]; // byte offset of (run g, pixel 0, column 0), OOB for a run beyond the last
        int px_left[4];      // pixels of run g inside the row
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (g > 0) {
                xr0 += 2;
                while (xr0 >= p.xt) {
                    xr0 -= p.xt;
                    ++line0;
                }
            }
            const bool r_ok = tile * 8 + 2 * g + fh < p.runs;
            pix_off[g] = (uint32_t)((line0 * p.ow + xr0 * TX) * p.N) * 4u;
            px_left[g] = r_ok ? p.ow - xr0 * TX : 0;
        }
#pragma unroll
        for (int i = 0; i < CT; ++i) {
            const int ncol = i * 32 + fr;
            const bool n_ok = ncol < p.N;
            const float bcol = (p.pw_b && n_ok) ? p.pw_b[ncol] : 0.f;
            float v[16];
            uint32_t off[16];
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    off[g * 4 + e] = (n_ok && e < px_left[g]) ? pix_off[g] + (uint32_t)(e * p.N + ncol) * 4u : OOB;
                    v[g * 4 + e] = acc[i][g * 4 + e] + bcol;
                }
            if (p.residual) {
#pragma unroll
                for (int z = 0; z < 16; ++z)
                    v[z] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srd_res, (int)off[z], 0, 0));
            }
            apply_act_block(v, p.act2);
#pragma unroll
            for (int z = 0; z < 16; ++z)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[z]), srd_out, (int)off[z], 0, 16); // agent scope: written through to memory, nothing left dirty in L2 at the kernel's end
        }
    }
}

// workgroups of `kernel` with `lds` bytes of dynamic LDS that are resident at once, remembered per (kernel, LDS size):
// the instantiations share one function type, so the table is keyed by the kernel's address (launches are serialised by
// the caller's stream order, the table by this mutex)
template <typename K>
static int64_t dwpw_resident(K kernel, size_t lds)
{
    static std::mutex mu;
    static std::map<std::pair<const void*, size_t>, int64_t> known;
    const std::pair<const void*, size_t> key(reinterpret_cast<const void*>(kernel), lds);
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find(key);
    if (it != known.end())
        return it->second;
    int per_cu = 1, dev = 0;
    hipDeviceProp_t prop;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, lds) != hipSuccess || per_cu < 1)
        per_cu = 1;
    const int cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) ? prop.multiProcessorCount : 256;
    return known[key] = (int64_t)per_cu * cus;
}

// LDS of a workgroup: the waves' A slabs, plus the whole 1x1 filter where that still leaves room for a second workgroup
static size_t dwpw_lds_bytes(int c, int n_out, bool* filter_in_lds)
{
    const int c_pad = (c + DWPW_KC - 1) / DWPW_KC * DWPW_KC, ct = (n_out + 31) / 32;
    const size_t slabs = sizeof(float) * 4 * 32 * DWPW_AS, filter = sizeof(float) * (size_t)ct * 32 * (c_pad + 4);
    *filter_in_lds = slabs + filter <= 64 * 1024;
    return slabs + (*filter_in_lds ? filter : 0);
}

static bool al16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

} // namespace fdx

using namespace fdx;

extern "C" int fdx_dwconv_pointwise_supported(int c, int n_out, int stride)
{
    return c > 0 && c % 4 == 0 && n_out > 0 && n_out <= DWPW_NP && (stride == 1 || stride == 2)
        && (int64_t)n_out * c * 4 < (1LL << 31);
}

extern "C" fdx_status fdx_dwconv_pointwise_nhwc_f32(const float* in, int n, int h, int w, int c, const float* dw_weights_hwc,
    const float* dw_bias, int stride, int pad_top, int pad_left, int out_h, int out_w, const fdx_act* dw_act,
    const float* pw_weights_nc, const float* pw_bias, int n_out, const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && dw_weights_hwc && pw_weights_nc && out, "dwconv_pointwise: null pointer");
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0, "dwconv_pointwise: bad shape");
    if (!fdx_dwconv_pointwise_supported(c, n_out, stride)) {
        set_error("dwconv_pointwise: needs channels %% 4 == 0, at most %d output channels and stride 1 or 2", DWPW_NP);
        return FDX_ERR_UNSUPPORTED;
    }
    FDX_REQUIRE_EPILOGUE_ACT(dw_act);
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(al16(in) && al16(dw_weights_hwc) && al16(pw_weights_nc) && (!dw_bias || al16(dw_bias)),
        "dwconv_pointwise: operands must be 16-byte aligned");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0 && (int64_t)(out_h - 1) * stride - pad_top < h
            && (int64_t)(out_w - 1) * stride - pad_left < w,
        "dwconv_pointwise: output size does not fit the input");
    DwPwParams p;
    p.in = in; p.dw_w = dw_weights_hwc; p.dw_b = dw_bias; p.pw_w = pw_weights_nc; p.pw_b = pw_bias; p.residual = residual; p.out = out;
    p.n = n; p.h = h; p.w = w; p.c = c; p.pad_top = pad_top; p.pad_left = pad_left; p.oh = out_h; p.ow = out_w; p.N = n_out;
    p.xt = (out_w + DWPW_TX - 1) / DWPW_TX;
    FDX_FUSED_LIMIT((int64_t)n * out_h * p.xt < (1LL << 31) - 64, "dwconv_pointwise: too many output pixels for one launch");
    p.runs = n * out_h * p.xt;
    p.c_pad = (c + DWPW_KC - 1) / DWPW_KC * DWPW_KC;
    FDX_FUSED_LIMIT((int64_t)n * h * w * c * 4 < (1LL << 31), "dwconv_pointwise: input tensor beyond 2 GiB");
    p.in_bytes = (uint32_t)((int64_t)n * h * w * c * 4);
    FDX_FUSED_LIMIT((int64_t)n * out_h * out_w * n_out * 4 < (1LL << 31), "dwconv_pointwise: output tensor beyond 2 GiB");
    p.out_bytes = (uint32_t)((int64_t)n * out_h * out_w * n_out * 4);
    p.act1 = make_act(dw_act);
    p.act2 = make_act(act);
    const int ct = (n_out + 31) / 32;
    bool in_lds = false;
    const size_t lds = dwpw_lds_bytes(c, n_out, &in_lds);
    const int64_t tiles = ((int64_t)p.runs + 7) / 8;
    // persistent waves: exactly the workgroups that are resident at once (a second round would run on a part of the chip)
    const int64_t want = (tiles + 3) / 4;
    profile_begin();
#define FDX_DWPW_L(S_, CT_, L_)                                                                              \
    {                                                                                                        \
        const int64_t resident = dwpw_resident(dwpw_kernel<S_, CT_, L_>, lds);                               \
        const unsigned grid = (unsigned)(want < resident ? want : resident);                                 \
        hipLaunchKernelGGL((dwpw_kernel<S_, CT_, L_>), dim3(grid), dim3(256), lds, stream(), p);             \
    }
#define FDX_DWPW(S_, CT_)                                                                                    \
    {                                                                                                        \
        if (in_lds)                                                                                          \
            FDX_DWPW_L(S_, CT_, true)                                                                        \
        else                                                                                                 \
            FDX_DWPW_L(S_, CT_, false)                                                                       \
    }
    if (stride == 1) {
        if (ct == 1) FDX_DWPW(1, 1) else if (ct == 2) FDX_DWPW(1, 2) else FDX_DWPW(1, 3)
    } else {
        if (ct == 1) FDX_DWPW(2, 1) else if (ct == 2) FDX_DWPW(2, 2) else FDX_DWPW(2, 3)
    }
#undef FDX_DWPW
#undef FDX_DWPW_L
    const double pix_in = (double)n * h * w, pix_out = (double)n * out_h * out_w;
    profile_end("dwconv_pointwise_f32", 2.0 * pix_out * c * n_out,
        4.0 * (pix_in * c + pix_out * n_out * (residual ? 2.0 : 1.0) + 9.0 * c + (double)n_out * c));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}
